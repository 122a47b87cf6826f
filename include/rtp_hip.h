/*
 * rtp_hip.h - C ABI of librtp_hip.so: gfx950 (MI355X) kernels for RTP's rotated-shard layer compute.
 *
 * The reference (wdlctc/rtp) has no FFI: its "operators" are the ATen calls made inside each
 * per-shard nn.Module.forward plus torch.distributed.batch_isend_irecv for the ring.  Every entry
 * point below names the reference call site (path:line under the reference tree) it stands in for.
 *
 * Conventions
 *  - every function returns 0 on success and a negative rtp_status on failure; the message of the
 *    last failure on the calling thread is returned by rtp_last_error().
 *  - all pointers are borrowed device pointers (the caller owns the memory and keeps it alive until
 *    the work queued on `stream` has completed).  Nothing here allocates device memory: ops that
 *    need scratch take a caller-provided workspace sized by the matching *_workspace_bytes().
 *  - every call is asynchronous on `stream` (a hipStream_t passed as void*); no call synchronises
 *    the device.
 *  - dtype: RTP_F32 or RTP_BF16 is the storage type of activations/weights; accumulation is fp32.
 */
#ifndef RTP_HIP_H
#define RTP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { RTP_F32 = 0, RTP_BF16 = 1 } rtp_dtype;

typedef enum {
  RTP_OK = 0,
  RTP_ERR_ARG = -1,     /* bad shape / null pointer / unsupported combination */
  RTP_ERR_DEVICE = -2,  /* current device is not gfx950 */
  RTP_ERR_HIP = -3,     /* a HIP runtime call failed */
  RTP_ERR_WORKSPACE = -4 /* workspace too small */
} rtp_status;

const char* rtp_last_error(void);

/* Version of this ABI (bumped on any signature change). */
int rtp_abi_version(void);

/* 0 if the current HIP device is gfx950, RTP_ERR_DEVICE otherwise.  `name_out` (optional, >= 64
 * bytes, host memory) receives the gcnArchName. */
int rtp_device_check(char* name_out, int name_len);

/* ---------------------------------------------------------------------------------------------
 * One rotated column-parallel Linear, all shards, one launch per product (reference: the per-layer ring loop of
 * ColumnParallelLinear.forward, rtp/module/linear.py:211-222 -- fetch the next shard, multiply, concatenate -- and its
 * backward through _WeightParallelRegion_before/_after, rtp/module/collectives.py:264-317).  The layer is described by
 * where its shards live: `home` is [shards, numel] flat shard buffers in `dtype` (shard g at home + g * numel), each
 * holding the weight [n_s, k] at element w_off and, if bias_off >= 0, the bias [n_s] there.  The product kernel
 * walks (shard, tile) work items in the ring order of rank 0 and streams every shard straight from home through
 * its LDS stages: nothing is copied or staged in device memory.
 *   fwd: y[rows, shards * n_s] (column block g) = x[rows, k] W_g^T + b_g; flags: RTP_GEMM_RELU (through a ReLU),
 *        RTP_GEMM_OUT_F32 (y is fp32 although the shards are bf16).
 *   bwd: either half may be left out (dx == NULL / grads == NULL), so that the two can go to different streams.
 *        dx[rows, k] = (dx_init +) sum_g dy[:, block g] W_g, optionally masked by relu_gate > 0 (the layer's input
 *        when it came out of a ReLU); dx_flags: RTP_GEMM_OUT_F32 / RTP_GEMM_CIN_F32 when dx / dx_init are fp32
 *        running sums of a layer whose shards arrive in several runs; grads is [shards, numel] like home: weight gradient dy[:, block g]^T x at
 *        w_off and the bias gradient at bias_off of row g, added to what is there when `accumulate`.  sgd_master /
 *        sgd_weights ([shards, numel] fp32 / `dtype`, laid out like home) ask for the clip + SGD update of rtp_gemm's
 *        fused epilogue; sgd_skip_grad_store then leaves the weight gradient unwritten.  colsum_workspace is only
 *        read when the bias gradient cannot ride in the weight-gradient launch (rtp_colsum_workspace_bytes(rows,
 *        shards * n_s) bytes).  What operands of odd alignment could not get is reported instead of refused when
 *        `done` (host memory, may be NULL) is given: it receives RTP_ROTATED_BIAS_DONE if the bias gradient was
 *        produced (always, given a workspace) and RTP_ROTATED_SGD_DONE if the update was applied; the caller then
 *        does the missing part itself (rtp_colsum, rtp_sgd_step).  Without `done` a part that cannot be done is
 *        an error.
 * --------------------------------------------------------------------------------------------- */
typedef struct {
  const void* home;
  int64_t numel, shards;
  int64_t w_off, bias_off; /* bias_off < 0: no bias */
  int64_t n_s, k;
} rtp_rotated_linear;

typedef struct {
  void* dx; /* may be NULL */
  int64_t ld_dx;
  const void* dx_init; /* may be NULL */
  int64_t ld_dx_init;
  const void* relu_gate; /* may be NULL */
  int64_t ld_relu_gate;
  int64_t dx_flags;
  void* grads; /* may be NULL */
  int32_t accumulate, sgd_skip_grad_store;
  void* sgd_master;  /* may be NULL */
  void* sgd_weights; /* may be NULL */
  float sgd_lr, sgd_clip;
  void* colsum_workspace; /* may be NULL */
  size_t colsum_workspace_bytes;
  int32_t* done; /* may be NULL */
} rtp_rotated_linear_bwd_args;
enum { RTP_ROTATED_BIAS_DONE = 1, RTP_ROTATED_SGD_DONE = 2 };

int rtp_rotated_linear_fwd(void* stream, int dtype, const rtp_rotated_linear* layer, const void* x, int64_t ldx,
                           int64_t rows, void* y, int64_t ldy, int flags);
int rtp_rotated_linear_bwd(void* stream, int dtype, const rtp_rotated_linear* layer, const void* dy, int64_t ldy,
                           const void* x, int64_t ldx, int64_t rows, const rtp_rotated_linear_bwd_args* args);

/* The logits layer together with its loss (reference: LinearLayer, rtp/models/transformer_lm_rtp.py:214-228, feeding
 * nn.CrossEntropyLoss()(output.view(-1, ntokens), targets), benchmarks/rtp_benchmark.py:182): the [rows, classes]
 * logits never reach memory.
 *   xent_fwd: loss[r] and stats[r] = {max, sum exp} of row r's logits x[r] W^T + b over all shards (fp32 [rows],
 *        fp32 [rows, 2]); loss and ignore_index as rtp_softmax_xent_fwd.  The logits product's epilogue leaves the
 *        statistics of every 64-column block in the workspace (rtp_rotated_linear_xent_workspace_bytes, 8-byte
 *        aligned) and a second small kernel combines them.  Feed loss to rtp_softmax_xent_reduce for a mean.
 *   xent_bwd: dlogits[rows, classes] = (softmax - onehot(target)) * dloss[0] * scale[0] (scale may be NULL), from
 *        the same product run once more with the row statistics; hand dlogits to rtp_rotated_linear_bwd as dy.
 * A shard's column count n_s must be a multiple of 64; operands vector-aligned as for the fused update. */
size_t rtp_rotated_linear_xent_workspace_bytes(const rtp_rotated_linear* layer, int64_t rows);
int rtp_rotated_linear_xent_fwd(void* stream, int dtype, const rtp_rotated_linear* layer, const void* x, int64_t ldx,
                                int64_t rows, const int64_t* target, int64_t ignore_index, float* loss, float* stats,
                                void* workspace, size_t workspace_bytes);
int rtp_rotated_linear_xent_bwd(void* stream, int dtype, const rtp_rotated_linear* layer, const void* x, int64_t ldx,
                                int64_t rows, const int64_t* target, int64_t ignore_index, const float* stats,
                                const float* dloss, const float* scale, void* dlogits, int64_t ld_dlogits);

/* ---------------------------------------------------------------------------------------------
 * GEMM   C[z][m,n] = epilogue( alpha * sum_k A[z](m,k) * B[z](n,k) )
 *
 * Stands in for F.linear inside the shard modules (rtp/module/linear.py:216, :385;
 * rtp/module/functional.py:303-308 in-projection, :798/:828 out-projection; rtp/module/top2gate.py:202
 * gate projection; rtp/models/transformer_lm_rtp.py:74-75 expert FFN), for the autograd backward
 * of those calls (dX = dY W, dW = dY^T X), and for the batched q k^T / p v products of
 * rtp/module/functional.py:779-792.
 *
 *   a_kcontig = 1 : A(m,k) is read at A[m*lda + k]       (row-major M x K)
 *   a_kcontig = 0 : A(m,k) is read at A[k*lda + m]       (stored K x M)
 *   b_kcontig = 1 : B(n,k) is read at B[n*ldb + k]       (row-major N x K, i.e. a torch Linear weight)
 *   b_kcontig = 0 : B(n,k) is read at B[k*ldb + n]       (stored K x N)
 *
 * Batching: grid z in [0, batch); z is split as zo = z / zdiv, zi = z % zdiv and every operand
 * pointer advances by zo*stride_o + zi*stride_i elements (so a (batch, head) pair can index a
 * packed [L, N, 3E] projection without a re-layout).
 *
 * Several rotation shards in one launch (what the reference does as a Python loop of ws small
 * matmuls, rtp/module/linear.py:211-220, :379-392):
 *   groups: `groups` independent problems of identical shape; group g advances every operand by
 *           g*stride_g elements (shard g's weight/bias in the flat shard buffer, its output column
 *           block, ...).  Replaces the per-shard F.linear + torch.cat of a column-parallel layer.
 *   ksegs:  the contraction is the concatenation of `ksegs` segments of length k; segment s reads A
 *           at a + s*a_sk and B at b + s*b_sk.  Replaces the `output + output_parallel` running sum
 *           over shards of row-parallel layers and the autograd sum of input gradients; the sum is
 *           kept in the fp32 MFMA accumulators.  If bias_sk != 0 the epilogue adds one bias per
 *           segment (bias + s*bias_sk), as every row-parallel shard carries bias/ws.
 *
 * Epilogue, in this order:  v = alpha*acc;  if c_in: v += c_in[m,n];  if bias: v += bias[n];
 * if RTP_GEMM_RELU: v = max(v,0);  if gate: v = gate[m,n] > 0 ? v : 0;  store to c_out as fp32
 * (RTP_GEMM_OUT_F32) or as `dtype`.  c_in is read as fp32 when RTP_GEMM_CIN_F32 is set, else as
 * `dtype`.  bias and gate are `dtype`.  c_in may alias c_out.
 *
 * Bias gradient from the same launch (a_rowsum != NULL): a_rowsum[group*rowsum_sg + m] = sum over the
 * whole contraction of A(m, k), in fp32 with a fixed order, stored as `dtype` (added to the existing value
 * with RTP_GEMM_ROWSUM_ACCUM).  In the weight-gradient product dW = dY^T X the operand A is dY^T, so this
 * is nn.Linear's bias gradient (reference: autograd of rtp/module/linear.py:216) without a second pass
 * over dY.  Only for descriptors rtp_gemm_rowsum_fused() accepts (A stored K x M, batch == 1, and the
 * alignment the wave-specialised kernel needs); rtp_gemm rejects others, callers use rtp_colsum there.
 * --------------------------------------------------------------------------------------------- */
enum {
  RTP_GEMM_OUT_F32 = 1,
  RTP_GEMM_CIN_F32 = 2,
  RTP_GEMM_RELU = 4,
  RTP_GEMM_STREAM_OUT = 8, /* c_out is not read again soon (weight gradients): non-temporal stores */
  RTP_GEMM_ROWSUM_ACCUM = 16, /* a_rowsum is added to, not overwritten */
  RTP_GEMM_SGD_SKIP_OUT = 32  /* with sgd_master: the product is consumed by the update, c_out is not written */
};

typedef struct {
  const void* a;
  const void* b;
  void* c_out;
  const void* c_in;  /* may be NULL */
  const void* bias;  /* may be NULL; length N */
  const void* gate;  /* may be NULL; same indexing as c_out but with ld_gate */
  int64_t m, n, k;
  int64_t lda, ldb, ldc, ld_cin, ld_gate;
  int64_t batch, zdiv; /* batch >= 1, zdiv >= 1 */
  int64_t a_so, a_si, b_so, b_si, c_so, c_si, cin_so, cin_si, gate_so, gate_si, bias_so, bias_si;
  int64_t groups, ksegs; /* >= 1 */
  int64_t a_sg, b_sg, c_sg, cin_sg, gate_sg, bias_sg; /* per-group element strides */
  int64_t a_sk, b_sk, bias_sk;                        /* per-K-segment element strides */
  float alpha;
  int32_t flags;
  int32_t a_kcontig, b_kcontig;
  void* a_rowsum;    /* may be NULL; length M per group */
  int64_t rowsum_sg; /* per-group element stride of a_rowsum */
  /* Clip + SGD applied to the product where it is produced (a weight-gradient product whose result would only be
   * read once more, by the optimiser: benchmarks/rtp_benchmark.py:185-186).  sgd_master (may be NULL: no update) is
   * the fp32 parameter buffer, sgd_weights (may be NULL) the `dtype` copy of it that the layers read; both are
   * indexed exactly like c_out (ldc, c_so, c_si, c_sg).  Per element: g = the product rounded to `dtype` (what
   * c_out receives), clamped to +-sgd_clip if sgd_clip > 0; master -= sgd_lr * g (product and difference rounded
   * separately, as rtp_sgd_step does); weights = master rounded to `dtype`.  Results are bit-identical to rtp_gemm
   * followed by rtp_sgd_step.  Needs vector-aligned operands, an output in `dtype` and a plain epilogue (no c_in,
   * bias, ReLU or gate); ask rtp_gemm_sgd_fused whether a descriptor qualifies. */
  void* sgd_master;
  void* sgd_weights;
  float sgd_lr, sgd_clip;
  /* Softmax cross-entropy over the rows of the product, for a product that is the logits of a column-parallel layer
   * (groups of n columns side by side, n a multiple of 64): what rtp_rotated_linear_xent_fwd / _bwd set up.
   * xent_mode 1: instead of the logits, {max, sum exp} of every 64-column block go to xent_part [m][groups*n/64] (pairs
   * of floats) and the logit of target[row] to xent_tlogit [m].  xent_mode 2: the logits are turned into
   * (softmax - onehot(target)) * xent_dloss[0] * xent_scale[0] before they are stored, with xent_stats [m] = {max,
   * sum exp} of each whole row; rows whose target equals xent_ignore (or lies outside the classes) get zeros. */
  int32_t xent_mode, xent_reserved;
  const int64_t* xent_target;
  int64_t xent_ignore;
  float* xent_part;
  float* xent_tlogit;
  const float* xent_stats;
  const float* xent_dloss;
  const float* xent_scale; /* may be NULL */
} rtp_gemm_desc;

int rtp_gemm(void* stream, int dtype, const rtp_gemm_desc* d);

/* "The next shard arrives while the current one computes" (reference: the irecv of the next shard under the current
 * step's product, rtp/module/linear.py:211-220, rtp/module/collectives.py:240-317) for shards that are read from
 * their home rows: hands `bytes` at `src` (16-byte aligned; the shards of the layer that runs next) to the next
 * product that this host thread launches through rtp_gemm or rtp_rotated_linear_* on the wave-specialised kernel.
 * That launch requests them at its start, so they sit in the GPU's memory-side cache when their own products run
 * (weights are read once per pass and would otherwise come from HBM at their turn).  Up to 192 KiB per workgroup
 * of the carrying launch.  A hint: no result depends on it; it ends with that next product launch whether or not
 * the launch could carry it (other kernels than the wave-specialised one cannot).  The carrying kernel reads `src` when
 * it RUNS, not when it is launched: `src` has to stay mapped until that launch has completed on its stream.  bytes == 0 withdraws a pending hint. */
int rtp_gemm_warm_next(const void* src, size_t bytes);

/* Measurement aid (no counterpart in the reference; bench.py reports it beside the published peak): TFLOP/s of a
 * register-only loop of v_mfma_f32_32x32x16_bf16 on every SIMD of the device, `iters` iterations of 32 MFMAs per
 * wavefront, with constant operands (random_operands == 0) or normally distributed ones (1).  Synchronises on
 * `stream`; allocates and frees 4 bytes. */
int rtp_probe_mfma_rate(void* stream, int random_operands, int iters, double* tflops);

/* 1 if rtp_gemm would produce d->a_rowsum for this descriptor (the pointer itself may still be NULL), else 0. */
int rtp_gemm_rowsum_fused(int dtype, const rtp_gemm_desc* d);

/* 1 if rtp_gemm would apply the fused update (sgd_master, sgd_weights) for this descriptor, else 0 (rtp_gemm then
 * refuses a descriptor that asks for it). */
int rtp_gemm_sgd_fused(int dtype, const rtp_gemm_desc* d);

/* sizeof(rtp_gemm_desc) as this library was compiled: lets a binding verify its struct layout. */
size_t rtp_gemm_desc_size(void);

/* Column sums in fp32 with a fixed summation order (deterministic): the bias gradient of nn.Linear's
 * backward (reference: autograd of rtp/module/linear.py:216).  Column c of x[m, n] (leading
 * dimension ld) is written to out[(c / seg) * seg_stride + c % seg], so the bias gradients of all
 * shards of a layer (seg columns each, seg_stride apart in the flat gradient buffer) come from one
 * call; seg <= 0 means one contiguous segment.  out is fp32 if out_f32 else `dtype`; accumulate != 0
 * adds to the existing contents.  workspace: rtp_colsum_workspace_bytes(m, n) bytes, 256-aligned. */
size_t rtp_colsum_workspace_bytes(int64_t m, int64_t n);
int rtp_colsum(void* stream, int dtype, const void* x, int64_t m, int64_t n, int64_t ld, void* out,
               int out_f32, int accumulate, int64_t seg, int64_t seg_stride, void* workspace,
               size_t workspace_bytes);

/* ---------------------------------------------------------------------------------------------
 * Shard rotation (reference: rtp/module/collectives.py:202-257 _left/_right_shift_buffer +
 * _WeightParallelRegion_before/after; rtp/rotated_tensor_parallel.py:114-151).  On one GPU the
 * isend/irecv pair of a ring step becomes a device-to-device copy of the next flat shard into the
 * spare slot of a two-slot staging buffer, queued on a side stream so it overlaps the compute
 * that is consuming the other slot.
 *
 * rtp_ring_create makes the side stream and the fencing events (no device memory).
 *   prefetch(main, slot, dst, src, n)  side stream: wait until the last consumer of `slot` released
 *                                it, copy.  May be called several times per slot before acquire.
 *                                A copy depends only on its slot, so the shards of the NEXT layer
 *                                stream in while the current layer still computes.
 *   acquire(main, slot)          main waits for the copies into `slot`
 *   release(main, slot)          marks the point on main after which `slot` may be overwritten
 *   fence(main)                  the shards' home storage is modified by work queued on main up to
 *                                here (optimizer step, weight load): the next prefetch waits for it.
 *                                The first prefetch after create behaves as if fenced.
 * Every copy is followed by an acquire on main, so the side stream is always joined back: a
 * sequence may be recorded into a HIP graph by capturing main (the side stream is forked from main
 * automatically when main is capturing).  After a capture ends, call fence before eager use.
 * --------------------------------------------------------------------------------------------- */
int rtp_ring_create(void** ring_out);
int rtp_ring_destroy(void* ring);
int rtp_ring_fence(void* ring, void* main_stream);
int rtp_ring_prefetch(void* ring, void* main_stream, int slot, void* dst, const void* src, size_t bytes);
int rtp_ring_acquire(void* ring, void* main_stream, int slot);
int rtp_ring_release(void* ring, void* main_stream, int slot);

/* Reads `bytes` at `src` (16-byte aligned) on `stream` and keeps nothing, so that the lines sit in the GPU's
 * memory-side cache when the products that use them start: the one-GPU form of "the next shard arrives while the
 * current one computes" (reference: the isend/irecv of the next shard that overlaps the current step's compute,
 * rtp/module/collectives.py:240-317, rtp/module/linear.py:211-220) when the shards are read from their home rows
 * and nothing is copied.  A hint: no result depends on it.  flags bit 0: non-temporal loads (measured: those do not
 * leave the lines in the memory-side cache, so the products that follow gain nothing; kept for such measurements). */
int rtp_cache_warm(void* stream, const void* src, size_t bytes, int flags);

/* The copy kernel on its own (16-byte vectorised, grid-stride): dst/src 16-byte aligned or any
 * alignment (falls back to bytes for the ragged ends). */
int rtp_shard_copy_async(void* stream, void* dst, const void* src, size_t bytes);

/* dst[i] = 0 for `bytes` bytes; a fill kernel (safe to record into a HIP graph). */
int rtp_zero_async(void* stream, void* dst, size_t bytes);

/* ---------------------------------------------------------------------------------------------
 * Embedding (reference: F.embedding at rtp/module/embedding.py:146 and its dense backward).
 * A shard is the rectangle rows [row_begin, row_begin+row_count) x `cols` columns of the master
 * table, stored row-major with leading dimension ld_table; the reference shards columns
 * (embedding.py:65-71) and uses row_begin = 0, row_count = V.
 *   gather:      out[t, 0:cols] = table[ids[t] - row_begin, 0:cols]   (ids outside the row range
 *                leave out[t] untouched); out has leading dimension ld_out.  `groups` shards are
 *                gathered by one launch: shard g reads table + g*table_sg, writes out + g*out_sg.
 *   scatter-add: grad_table[ids[t] - row_begin, :] += grad_out[t, :]  summed per row in ascending t
 *                (sequential fp32 adds starting from +0.0f: bit-identical to torch's CPU
 *                nn.Embedding backward / index_add_).  Rows that receive no token are zero-filled
 *                when zero_fill != 0.  Tokens equal to padding_idx (if >= 0) are skipped.
 *                When scale_by_freq != 0 each row's sum is divided by the number of tokens that
 *                hit it.  `groups` shards in one launch: shard g reads grad_out + g*grad_out_sg and
 *                writes grad_table + g*grad_table_sg (elements).
 * ids are int64.  The scatter-add needs a workspace (sort buffers).
 * --------------------------------------------------------------------------------------------- */
int rtp_embedding_gather(void* stream, int dtype, const void* table, int64_t ld_table,
                         int64_t row_begin, int64_t row_count, int64_t cols, const int64_t* ids,
                         int64_t n_ids, void* out, int64_t ld_out, int64_t groups, int64_t table_sg,
                         int64_t out_sg);

/* The gather fused with the two element-wise steps the language model applies to it (reference:
 * rtp/models/transformer_lm_rtp.py:27-28 `embedding(src) * sqrt(ninp)` and :49 `x + pe[:x.size(0)]`):
 *   out[t, c] = T( T(table[ids[t], c] * scale) + pos[t / batch, c] ), each step rounded to the element type as
 * the separate operations round.  Tokens are laid out [sequence, batch] so t / batch is the position; shard g reads
 * the positional table at pos + g*pos_sg (leading dimension ld_pos). */
int rtp_embedding_gather_scale_pos(void* stream, int dtype, const void* table, int64_t ld_table,
                                   int64_t row_begin, int64_t row_count, int64_t cols, const int64_t* ids,
                                   int64_t n_ids, void* out, int64_t ld_out, int64_t groups, int64_t table_sg,
                                   int64_t out_sg, float scale, const void* pos, int64_t ld_pos, int64_t pos_sg,
                                   int64_t batch);

size_t rtp_embedding_scatter_workspace_bytes(int64_t n_ids);

/* Sorts (id, position) once; the result in `workspace` is reused by every shard of the layer. */
int rtp_embedding_sort_ids(void* stream, const int64_t* ids, int64_t n_ids, void* workspace,
                           size_t workspace_bytes);

int rtp_embedding_scatter_add_det(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out,
                                  int64_t n_ids, const void* workspace, void* grad_table,
                                  int64_t ld_grad_table, int grad_table_f32, int64_t row_begin,
                                  int64_t row_count, int64_t cols, int64_t padding_idx,
                                  int scale_by_freq, int zero_fill, int64_t groups, int64_t grad_out_sg,
                                  int64_t grad_table_sg);

/* Backward of rtp_embedding_gather_scale_pos: the same ordered sum over T(grad_out[t, :] * grad_scale), the
 * gradient the multiplication by the scale hands to the embedding (transformer_lm_rtp.py:27-28). */
int rtp_embedding_scatter_add_scaled(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out,
                                     int64_t n_ids, const void* workspace, void* grad_table,
                                     int64_t ld_grad_table, int grad_table_f32, int64_t row_begin,
                                     int64_t row_count, int64_t cols, int64_t padding_idx,
                                     int scale_by_freq, int zero_fill, int64_t groups, int64_t grad_out_sg,
                                     int64_t grad_table_sg, float grad_scale);

/* rtp_embedding_scatter_add_scaled with the optimiser's update applied where a row's gradient is produced
 * (reference: the embedding's share of `clip_grad_value_` + `optimizer.step()`, benchmarks/rtp_benchmark.py:185-186,
 * for plain SGD): every table row some token names gets w = master - lr * clamp(T(sum), +-clip) (clip == 0: no
 * clamp), the arithmetic of rtp_sgd_step on the gradient as its table would hold it; `weights` (may be NULL) receives
 * the row in `dtype`.  master is fp32, laid out like grad_table (same leading dimension and group stride).  Rows no
 * token names have a zero gradient, which the update leaves unchanged: they are not touched, and with
 * store_grad == 0 the dense gradient table is neither filled nor written.  The caller guarantees one backward pass
 * per update (the sum is the row's whole gradient). */
int rtp_embedding_scatter_add_sgd(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out, int64_t n_ids,
                                  const void* workspace, void* grad_table, int64_t ld_grad_table, int64_t row_begin,
                                  int64_t row_count, int64_t cols, int64_t padding_idx, int scale_by_freq,
                                  int64_t groups, int64_t grad_out_sg, int64_t grad_table_sg, float grad_scale,
                                  float* master, void* weights, float lr, float clip, int store_grad);

/* The backward of F.embedding in ONE launch, straight from the token ids (reference: the autograd backward of
 * rtp/module/embedding.py:146, there a dense zeros + index_add_ per shard): the arguments and results of
 * rtp_embedding_scatter_add_scaled / _sgd (same order of summation, bit for bit) without the sort and without a
 * separate fill.  Every workgroup keeps the step's ids in LDS; the workgroup of token position t sums the upstream rows
 * of all positions that name the same id, ascending, if t is the first of them, for all `groups` shards; with
 * zero_fill the rows that no token names are cleared by further workgroups of the same launch.  master == NULL: the
 * gradient is written (zero_fill != 0: overwriting, else added to what is there); master != NULL: the update of
 * rtp_embedding_scatter_add_sgd (weights may be NULL; store_grad as there).  At most 4096 ids
 * (rtp_embedding_backward_supported); longer steps take rtp_embedding_sort_ids + rtp_embedding_scatter_add_*. */
int rtp_embedding_backward_supported(int64_t n_ids);
int rtp_embedding_backward(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out, int64_t n_ids,
                           const int64_t* ids, void* grad_table, int64_t ld_grad_table, int grad_table_f32,
                           int64_t row_begin, int64_t row_count, int64_t cols, int64_t padding_idx, int scale_by_freq,
                           int zero_fill, int64_t groups, int64_t grad_out_sg, int64_t grad_table_sg, float grad_scale,
                           float* master, void* weights, float lr, float clip, int store_grad);

/* ---------------------------------------------------------------------------------------------
 * Attention softmax (reference: rtp/module/functional.py:779-792 baddbmm+softmax, :825
 * scaled_dot_product_attention with an additive float mask).
 *   fwd: p[z,i,j] = softmax_j( scale*s[z,i,j] + mask[i,j] + key_bias[b,j] )  (and j <= i + (S-L) only, if causal)
 *        s fp32 [Z,L,S] contiguous, mask fp32 [L,S] or NULL, p `dtype` [Z,L,S]; key_bias fp32 [n_batch,S] or NULL is
 *        the key padding mask (0 / -inf, functional.py:760-768 merges it into the mask per batch), with
 *        z = (group * n_batch + b) * heads + head.
 *   bwd: ds[z,i,j] = scale * p * (dp - sum_j dp*p)           dp fp32, ds `dtype`.
 * Attention dropout (functional.py:789-792 / the dropout_p of :825): `keep` fp32 [Z,L,S] holds 0 or 1 / (1 - rate) per
 * probability (the draw is the caller's).  fwd then also writes p_dropped = p * keep, the operand of the product with
 * V; bwd takes dp as the gradient of p_dropped and multiplies it by keep first.  Both NULL: no dropout.
 * One wavefront per row, fp32 max/sum by cross-lane reduction.
 * --------------------------------------------------------------------------------------------- */
int rtp_softmax_fwd(void* stream, int dtype, const float* s, const float* mask, const float* key_bias,
                    int64_t n_batch, int64_t heads, int causal, float scale, int64_t z, int64_t l, int64_t skv,
                    void* p);
/* The same with one mask per problem (the 3-D attn_mask [batch * heads, L, S] of functional.py:701-704): mask is fp32
 * [mask_problems, L, S] and problem z takes mask[z % mask_problems]; mask_problems <= 1 is the single-mask form. */
int rtp_softmax_fwd_masks(void* stream, int dtype, const float* s, const float* mask, int64_t mask_problems,
                          const float* key_bias, int64_t n_batch, int64_t heads, int causal, float scale, int64_t z,
                          int64_t l, int64_t skv, void* p, const float* keep, void* p_dropped);
int rtp_softmax_bwd(void* stream, int dtype, const void* p, const float* dp, const float* keep, float scale,
                    int64_t z, int64_t l, int64_t skv, void* ds);

/* ---------------------------------------------------------------------------------------------
 * Fused attention core for short sequences (reference: the per-head-group core of
 * multi_head_attention_forward, rtp/module/functional.py:779-800 and :815-830: q k^T -> (+mask) softmax ->
 * p v, and its autograd backward).  bf16 only, L <= 32, head dimension D in {32, 64, 128}
 * (rtp_attn_supported says whether a shape qualifies; otherwise compose rtp_gemm + rtp_softmax_*).
 * One wavefront per (group, batch, head); scores and probabilities never leave registers except for the
 * stored p.  Element (l, b, h, g, dd) of q/k/v/dq/dk/dv is at base + l*s_l + b*s_b + h*s_h + g*s_g + dd, of
 * o/dout at base + l*o_l + b*o_b + h*o_h + g*o_g + dd (strides in elements, multiples of 8; bases 16-byte
 * aligned).  p is [G][N][H][L][L] bf16, written by fwd and read by bwd.  mask: additive fp32 [L][L] or
 * NULL; key_bias: additive fp32 [N][L] per (batch, key) or NULL (the key padding mask: 0 / -inf); causal != 0
 * hides keys j > i.  scale multiplies the scores before the masks are added.
 *   fwd: p = softmax(scale * q k^T + mask + key_bias), o = p v
 *   bwd: dv = p^T dout, dp = dout v^T, ds = scale * p o (dp - rowsum(dp o p)), dq = ds k, dk = ds^T q
 * --------------------------------------------------------------------------------------------- */
int rtp_attn_supported(int dtype, int64_t L, int64_t D);
int rtp_attn_fwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                 int64_t s_b, int64_t s_h, int64_t s_g, void* o, int64_t o_l, int64_t o_b, int64_t o_h,
                 int64_t o_g, void* p, const float* mask, const float* key_bias, int causal, float scale,
                 int64_t L, int64_t N, int64_t H, int64_t D, int64_t G);
int rtp_attn_bwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                 int64_t s_b, int64_t s_h, int64_t s_g, const void* dout, int64_t o_l, int64_t o_b,
                 int64_t o_h, int64_t o_g, const void* p, void* dq, void* dk, void* dv, float scale,
                 int64_t L, int64_t N, int64_t H, int64_t D, int64_t G);

/* ---------------------------------------------------------------------------------------------
 * Fused attention core for any sequence length (reference: the same per-head-group core,
 * rtp/module/functional.py:779-800 and :815-830, there bmm -> softmax -> bmm with the [L, L] probabilities
 * in memory).  bf16 only, D in {32, 64, 128}; addressing, mask, key_bias, causal and scale as for rtp_attn_fwd.  One
 * wavefront per (group, batch, head, 32-query block) walks the keys in blocks of 32 with a running softmax;
 * the probabilities are never stored.  lse and delta are fp32 [G][N][H][L].
 *   fwd: o = softmax(scale * q k^T + mask) v,  lse = log sum_j exp(scale * q k_j + mask_j)
 *   bwd: p recomputed from lse; delta = rowsum(dout o o) (written here, scratch for the caller);
 *        dv = p^T dout, ds = scale * p o (dout v^T - delta), dq = ds k, dk = ds^T q
 * A query whose keys are all masked with -inf gets o = 0 and lse = 0 (torch gives NaN there).
 * --------------------------------------------------------------------------------------------- */
int rtp_attn_flash_supported(int dtype, int64_t L, int64_t D);
int rtp_attn_flash_fwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                       int64_t s_b, int64_t s_h, int64_t s_g, void* o, int64_t o_l, int64_t o_b, int64_t o_h,
                       int64_t o_g, float* lse, const float* mask, const float* key_bias, int causal, float scale,
                       int64_t L, int64_t N, int64_t H, int64_t D, int64_t G);
int rtp_attn_flash_bwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                       int64_t s_b, int64_t s_h, int64_t s_g, const void* o, const void* dout, int64_t o_l,
                       int64_t o_b, int64_t o_h, int64_t o_g, const float* lse, float* delta, void* dq,
                       void* dk, void* dv, const float* mask, const float* key_bias, int causal, float scale,
                       int64_t L, int64_t N, int64_t H, int64_t D, int64_t G);

/* ---------------------------------------------------------------------------------------------
 * Residual add + LayerNorm of the post-LN decoder layer (reference: norm1(x + sa_block(x)) and
 * norm2(x + ff_block(x)), rtp/models/transformer_lm_rtp.py:176-177, there two ATen calls each way).
 *   fwd: z = x + r (rounded to `dtype`; r NULL: z = x, z_out unused), y = (z - mean) * rstd * gamma + beta,
 *        mean / rstd fp32 [rows].  z_out is what bwd needs.
 *   bwd: dz = rstd * (g - mean_c(g) - zhat * mean_c(g * zhat)), g = dy * gamma, zhat = (z - mean) * rstd;
 *        dgamma = sum_rows dy * zhat, dbeta = sum_rows dy (dbeta may be NULL); fixed summation order.
 * fp32 or bf16, rows contiguous, cols a multiple of 16 bytes and <= 2048 (rtp_layernorm_supported).
 * --------------------------------------------------------------------------------------------- */
int rtp_layernorm_supported(int dtype, int64_t cols);
int rtp_add_layernorm_fwd(void* stream, int dtype, const void* x, const void* r, const void* gamma,
                          const void* beta, float eps, int64_t rows, int64_t cols, void* z_out, void* y,
                          float* mean, float* rstd);
size_t rtp_layernorm_bwd_workspace_bytes(int64_t rows, int64_t cols);
int rtp_layernorm_bwd(void* stream, int dtype, const void* dy, const void* z, const void* gamma,
                      const float* mean, const float* rstd, int64_t rows, int64_t cols, void* dz,
                      void* dgamma, void* dbeta, void* workspace, size_t workspace_bytes);

/* Deferred parameter gradients: rtp_layernorm_bwd with dgamma == NULL writes dz and leaves the per-block partial
 * sums [rtp_layernorm_bwd_blocks(rows)][2][cols] (fp32) in `workspace`; rtp_layernorm_bwd_finalize then reduces the
 * partial sums of MANY LayerNorms (same dtype) in one launch -- a caller that only needs dgamma / dbeta when the
 * backward pass ends saves a launch per layer.  `items` is a table in DEVICE memory; max_cols = the widest entry. */
typedef struct {
  const float* part; /* the workspace of that layer's rtp_layernorm_bwd call */
  int64_t nblocks;   /* rtp_layernorm_bwd_blocks(rows) */
  int64_t cols;
  void* dgamma;
  void* dbeta; /* may be NULL */
} rtp_ln_final_item;
int64_t rtp_layernorm_bwd_blocks(int64_t rows);
int rtp_layernorm_bwd_finalize(void* stream, int dtype, const rtp_ln_final_item* items, int64_t n_items,
                               int64_t max_cols);

/* ---------------------------------------------------------------------------------------------
 * Softmax cross-entropy over the vocabulary axis of the LM's logits (reference harness:
 * nn.CrossEntropyLoss()(outputs.view(-1, vocab_size), labels.view(-1)), test_transformer.py:195-197,
 * there a log-softmax, a gather and their backward over an fp32 copy of the logits).
 *   fwd: stats[r] = {m, s}, m = max_j logits[r, j], s = sum_j exp(logits[r, j] - m) (fp32 [rows, 2]);
 *        loss[r] = (m - logits[r, target[r]]) + log s (fp32 [rows]).
 *   bwd: dlogits[r, j] = (exp(logits[r, j] - m) / s - [j == target[r]]) * dloss[r * dloss_stride] * scale[0],
 *        dloss fp32 (dloss_stride 0: one scalar for all rows, 1: one value per row); scale: a device scalar, may
 *        be NULL for 1.
 *   reduce: out[0] = sum_r loss[r], divided by the number of rows with target != ignore_index when `mean`;
 *        scale[0] = 1 / that number (1 without `mean`) -- the `scale` of the backward pass of a mean loss.  One
 *        workgroup, fixed summation order; no rows at all or all ignored gives NaN, as torch does.
 * A row whose target equals ignore_index (inside the class range or not: a padding id such as 0 counts) has loss 0
 * and gradient 0, in fwd, reduce and bwd alike.  Any other target outside [0, cols) is the
 * caller's error (torch asserts on the device): its loss is NaN, which shows in every sum over the rows, and its
 * gradient 0.  fp32 or bf16 logits, statistics in fp32.  Rows of whole 16-byte vectors (cols and both leading
 * dimensions multiples of 16 bytes, 16-byte aligned, at most 8192 vectors: 65536 bf16 or 32768 fp32 classes) are
 * held in registers and read once; anything else takes element-wise kernels with the same results.
 * dlogits may alias logits.
 * --------------------------------------------------------------------------------------------- */
int rtp_softmax_xent_fwd(void* stream, int dtype, const void* logits, int64_t ld, int64_t rows, int64_t cols,
                         const int64_t* target, int64_t ignore_index, float* loss, float* stats);
/* loss / stats of every row from the {max, sum exp} pairs of its 64-column blocks (part [rows, blocks] pairs) and the
 * target's logit tlogit [rows]: the second step of rtp_rotated_linear_xent_fwd. */
int rtp_softmax_xent_combine(void* stream, const float* part, int64_t blocks, const float* tlogit,
                             const int64_t* target, int64_t ignore_index, int64_t rows, float* loss, float* stats);
int rtp_softmax_xent_reduce(void* stream, const float* loss, const int64_t* target, int64_t ignore_index,
                            int64_t rows, int mean, float* out, float* scale);
int rtp_softmax_xent_bwd(void* stream, int dtype, const void* logits, int64_t ld, int64_t rows, int64_t cols,
                         const int64_t* target, int64_t ignore_index, const float* stats, const float* dloss,
                         int64_t dloss_stride, const float* scale, void* dlogits, int64_t ld_dlogits);

/* ---------------------------------------------------------------------------------------------
 * Top-2 routing (reference: top2gating, rtp/module/top2gate.py:43-105).
 * Inputs logits[S,E] fp32 and noise[S,E] fp32 (the Gumbel sample of top2gate.py:61, supplied by the
 * caller so that routing is a pure function of its inputs).  Outputs, per token s:
 *   expert[s,2] int32, slot[s,2] int32 (location in the expert's capacity buffer, 0 if dropped),
 *   keep[s,2] int32 (1 if the choice survived the capacity drop and has a non-zero weight),
 *   weight[s,2] fp32 (renormalised gate probabilities, 0 if dropped), gates[S,E] fp32 (softmax),
 *   slot_token[E*C] int32 (token occupying each capacity slot, -1 if empty), l_aux fp32 scalar,
 *   counts[2*E] int32 (first-choice and second-choice totals per expert before the drop).
 * capacity C = 2*S/E; requires S % E == 0 and E <= 64.  l_aux_bf16 (may be NULL): a bf16 copy of l_aux for a layer
 * that runs in bf16 (the reference returns l_aux in the logits' dtype, top2gate.py:105).
 * --------------------------------------------------------------------------------------------- */
size_t rtp_top2_route_workspace_bytes(int64_t s, int64_t e);
int rtp_top2_route(void* stream, const float* logits, const float* noise, int64_t s, int64_t e,
                   int32_t* expert, int32_t* slot, int32_t* keep, float* weight, float* gates,
                   int32_t* slot_token, float* l_aux, int32_t* counts, void* workspace,
                   size_t workspace_bytes, void* l_aux_bf16);

/* Backward of the differentiable part of top2gating: d_logits[S,E] from d_weight[S,2] and the
 * scalar d_l_aux (device pointer, may be NULL for 0). */
int rtp_top2_route_bwd(void* stream, const float* gates, const int32_t* expert, const int32_t* keep,
                       const int32_t* counts, const float* d_weight, const float* d_l_aux,
                       int64_t s, int64_t e, float* d_logits);

/* ---------------------------------------------------------------------------------------------
 * MoE dispatch / combine (reference: the dense einsums "sec,sm->ecm" rtp/module/moe.py:148 and
 * "sec,ecm->sm" :174, restated as row moves through the compact routing).
 *   dispatch: out[e*C + c, :] = x[slot_token[e*C+c], :] * (w ? w-of-that-choice : 1), 0 if empty.
 *             With weight == NULL this is the forward dispatch; with weight it is the backward of
 *             combine w.r.t. the expert outputs.
 *   combine:  out[s,:] = sum_{j<2, keep[s,j]} w[s,j] * y[expert[s,j]*C + slot[s,j], :]
 *             (weight == NULL means w = 1: the backward of dispatch).
 *   combine_dweight: dw[s,j] = keep[s,j] ? dot(dout[s,:], y[expert*C+slot, :]) : 0   (fp32).
 * --------------------------------------------------------------------------------------------- */
int rtp_moe_dispatch(void* stream, int dtype, const void* x, int64_t ld_x, const int32_t* slot_token,
                     const int32_t* expert, const int32_t* slot, const float* weight,
                     int64_t n_slots, int64_t capacity, int64_t cols, void* out, int64_t ld_out);
int rtp_moe_combine(void* stream, int dtype, const void* y, int64_t ld_y, const int32_t* expert,
                    const int32_t* slot, const int32_t* keep, const float* weight, int64_t s,
                    int64_t capacity, int64_t cols, void* out, int64_t ld_out);
int rtp_moe_combine_dweight(void* stream, int dtype, const void* dout, int64_t ld_dout, const void* y,
                            int64_t ld_y, const int32_t* expert, const int32_t* slot,
                            const int32_t* keep, int64_t s, int64_t capacity, int64_t cols,
                            float* dweight);

/* ---------------------------------------------------------------------------------------------
 * Gate projection with few experts (reference: `logits = self.wg(input)` of the rotated gate,
 * rtp/module/top2gate.py:195-207 -- an nn.Linear without bias whose expert rows are sharded -- and its autograd
 * backward).  With E <= 16 output columns these are streaming passes over the tokens, not tiled products:
 *   fwd:   logits[s][e] = sum_m x[s][m] * w[e][m]                  fp32 logits
 *   dgrad: dx[s][m]     = sum_e dlogits[s][e] * w[e][m]            fp32 dlogits, e ascending, rounded once; with
 *          dx_init (may be NULL; `dtype`, may alias dx) dx = dx_init + that, the sum autograd forms where the gradients
 *          of a tensor's two consumers meet (the MoE layer's tokens feed the gate and the dispatch, moe.py:146-148)
 *   wgrad: dw[e][m]   (+)= sum_s dlogits[s][e] * x[s][m]           partial sums of 64 token rows, then summed in order
 * x [S, M], w and dw [E, M] in `dtype` with element row pitches; rtp_gate_supported says whether (E, M) qualify
 * (E <= 16, M a multiple of 16 bytes); x, w, dx must be 16-byte aligned with pitches that keep rows so.  The rows
 * of w / dw of consecutive shards are consecutive rows of one matrix when a shard's flat buffer is exactly its
 * [E/ws, M] weight.  Otherwise use rtp_gemm.
 * --------------------------------------------------------------------------------------------- */
int rtp_gate_supported(int dtype, int64_t experts, int64_t model_dim);
int rtp_gate_fwd(void* stream, int dtype, const void* x, int64_t ldx, const void* w, int64_t ldw, int64_t S,
                 int64_t M, int64_t E, float* logits, int64_t ld_logits);
int rtp_gate_dgrad(void* stream, int dtype, const float* dlogits, int64_t ld_dlogits, const void* w, int64_t ldw,
                   int64_t S, int64_t M, int64_t E, void* dx, int64_t ldx, const void* dx_init, int64_t ld_dx_init);
size_t rtp_gate_wgrad_workspace_bytes(int64_t S, int64_t M, int64_t E);
int rtp_gate_wgrad(void* stream, int dtype, const float* dlogits, int64_t ld_dlogits, const void* x, int64_t ldx,
                   int64_t S, int64_t M, int64_t E, void* dw, int64_t ld_dw, int accumulate, void* workspace,
                   size_t workspace_bytes);

/* rtp_gate_wgrad for callers that cannot allocate (code under HIP-graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as rtp_gate_wgrad without the
 * workspace: the partial sums go to a buffer built into the library (RTP_GATE_WGRAD_STATIC_MAX_BYTES = 8 MiB of device
 * memory per GPU, held until the process ends), so ceil(S / 64) * E * M * 4 bytes must not exceed that size -- larger
 * problems are refused with RTP_ERR_ARG and belong to rtp_gate_wgrad.  The call allocates and frees nothing.  Every
 * call on a GPU uses that GPU's one buffer: calls that may overlap on one GPU (different streams) race; calls on one
 * stream, or ordered by events, do not.  Nothing in the buffer has to be cleared between calls. */
#define RTP_GATE_WGRAD_STATIC_MAX_BYTES ((size_t)8 << 20)
int rtp_gate_wgrad_static(void* stream, int dtype, const float* dlogits, int64_t ld_dlogits, const void* x,
                          int64_t ldx, int64_t S, int64_t M, int64_t E, void* dw, int64_t ld_dw, int accumulate);

/* ---------------------------------------------------------------------------------------------
 * Out-channel-sharded 2-D convolution (reference: the per-shard `self.layers[index](input_)` = F.conv2d of
 * ColumnParallelConv2d, rtp/module/conv.py:99-114, and its autograd backward) as an implicit GEMM: the patch matrix
 *   patches[(n*Ho+ho)*Wo+wo][(ci*kh+i)*kw+j] = x[n][ci][ho*sh-ph+i*dh][wo*sw-pw+j*dw]   (0 outside: zero padding)
 * is gathered by the product kernel as it goes and never written to memory (groups = 1).  A run of `shards`
 * consecutive shards is described like a rotated linear layer: `w` / `grads` point at the run's first shard row,
 * rows are `numel` elements apart, a shard's weight [n_s, Ci, kh, kw] (as stored: row-major [n_s, Ci*kh*kw]) sits at
 * element w_off of its row and its bias [n_s] at bias_off (bias_off < 0: none); the run produces / reads output
 * channels co_first .. co_first + shards*n_s - 1.  Activations x and dy are addressed by element strides (any memory
 * format); y and dx are contiguous NCHW.
 *   fwd:    y[n][co][ho][wo] = sum_k W[co][k] patches[pix][k] + b[co]; y has co_total channels in all
 *   wgrad:  grads_s[w_off + co*K + k] (+)= sum_pix dy[n][co][ho][wo] patches[pix][k], and with bias_off >= 0
 *           grads_s[bias_off + co] (+)= sum_pix dy[n][co][ho][wo]   (fp32 sums in a fixed order; (+) = accumulate != 0);
 *           the sum over the pixels is dealt over several workgroups whose fp32 partial sums go through `workspace`
 *           (rtp_conv2d_wgrad_workspace_bytes of device memory, 0 for small problems; 16-byte aligned)
 *   dgrad:  dx[n][ci][h][w] = addend + sum over the run's (co, i, j) of W[co][ci][i][j] dy[n][co][ho][wo] for the
 *           output pixels that read x[n][ci][h][w]; dx_f32 / addend_f32: that array is fp32 although dtype is bf16
 *           (the sum over several runs is kept in fp32 and rounded by the last one); addend may be NULL or dx itself
 * ho / wo must equal floor((h + 2*ph - dh*(kh-1) - 1) / sh) + 1 (and likewise for w).
 * --------------------------------------------------------------------------------------------- */
typedef struct {
  int64_t n, c, h, w;   /* input: batch, channels, height, width */
  int64_t kh, kw;       /* kernel */
  int64_t sh, sw;       /* stride */
  int64_t ph, pw;       /* zero padding on each side */
  int64_t dh, dw;       /* dilation */
  int64_t ho, wo;       /* output height, width */
} rtp_conv_geom;
int rtp_conv2d_fwd(void* stream, int dtype, const void* x, int64_t sx_n, int64_t sx_c, int64_t sx_h, int64_t sx_w,
                   const rtp_conv_geom* geom, const void* w, int64_t numel, int64_t shards, int64_t w_off,
                   int64_t bias_off, int64_t n_s, void* y, int64_t co_first, int64_t co_total);
int rtp_conv2d_wgrad(void* stream, int dtype, const void* dy, int64_t sdy_n, int64_t sdy_c, int64_t sdy_h,
                     int64_t sdy_w, const void* x, int64_t sx_n, int64_t sx_c, int64_t sx_h, int64_t sx_w,
                     const rtp_conv_geom* geom, void* grads, int64_t numel, int64_t shards, int64_t w_off,
                     int64_t bias_off, int64_t n_s, int64_t co_first, int accumulate, void* workspace,
                     size_t workspace_bytes);
size_t rtp_conv2d_wgrad_workspace_bytes(const rtp_conv_geom* geom, int64_t shards, int64_t n_s);
int rtp_conv2d_dgrad(void* stream, int dtype, const void* dy, int64_t sdy_n, int64_t sdy_c, int64_t sdy_h,
                     int64_t sdy_w, const rtp_conv_geom* geom, const void* w, int64_t numel, int64_t shards,
                     int64_t w_off, int64_t n_s, int64_t co_first, void* dx, int dx_f32, const void* addend,
                     int addend_f32);

/* ---------------------------------------------------------------------------------------------
 * Optimiser step on a flat shard buffer (reference harness: clip_grad_value_ + optimizer.step,
 * benchmarks/rtp_benchmark.py:185-186; SGD as the headline configuration asks).
 *   g = clamp(grad, -clip, clip) if clip > 0;  master -= lr * g;  shadow = (dtype) master.
 * master fp32; grad `dtype`; shadow `dtype` (may be NULL when dtype is fp32 and the master is the
 * weight itself).
 * --------------------------------------------------------------------------------------------- */
int rtp_sgd_step(void* stream, int dtype, float* master, const void* grad, void* shadow, int64_t n,
                 float lr, float clip);

/* Adam on a flat shard buffer (reference harness: clip_grad_value_(0.05) then torch.optim.Adam(lr 1e-3),
 * benchmarks/rtp_benchmark.py:41-42 and :185-186), torch.optim.Adam's arithmetic without amsgrad / maximize:
 *   g = clamp(grad, -clip, clip) if clip > 0;  g += weight_decay * master if weight_decay != 0
 *   exp_avg += (1 - beta1) * (g - exp_avg);  exp_avg_sq = beta2 * exp_avg_sq + (1 - beta2) * g * g
 *   master -= lr / (1 - beta1^step) * exp_avg / (sqrt(exp_avg_sq) / sqrt(1 - beta2^step) + eps)
 *   shadow = (dtype) master
 * master, exp_avg, exp_avg_sq fp32 (the state starts at zero, `step` counts from 1); grad and shadow `dtype`
 * (shadow may be NULL when dtype is fp32 and the master is the weight itself).  step_dev non-NULL: the step
 * count is read from this device location when the kernel runs and `step` is ignored, so that a launch
 * recorded into a HIP graph follows a counter the caller advances (on the same stream, before the launch). */
int rtp_adam_step(void* stream, int dtype, float* master, const void* grad, void* shadow, float* exp_avg,
                  float* exp_avg_sq, int64_t n, double lr, double beta1, double beta2, double eps,
                  double weight_decay, int64_t step, const int64_t* step_dev, double clip);

/* The same update for many buffers in one launch.  `chunks` is a table in DEVICE memory, one entry per
 * workgroup: 16-byte aligned pointers into the buffers and a parameter count that is a multiple of 4 (the
 * caller cuts its buffers into chunks of, say, 16384 parameters).  total_params only feeds the profiler. */
typedef struct {
  float* master;
  const void* grad;
  void* shadow; /* NULL: the master is the weight */
  int64_t n;
} rtp_sgd_chunk;
int rtp_sgd_step_multi(void* stream, int dtype, const rtp_sgd_chunk* chunks, int64_t n_chunks, float lr,
                       float clip, double total_params);

/* Adam for many buffers in one launch, like rtp_sgd_step_multi: `chunks` is a table in DEVICE memory, one entry per
 * workgroup (16-byte aligned pointers, a parameter count that is a multiple of 4); the other arguments as for
 * rtp_adam_step.  total_params only feeds the profiler. */
typedef struct {
  float* master;
  const void* grad;
  void* shadow; /* NULL: the master is the weight */
  float* exp_avg;
  float* exp_avg_sq;
  int64_t n;
} rtp_adam_chunk;
int rtp_adam_step_multi(void* stream, int dtype, const rtp_adam_chunk* chunks, int64_t n_chunks, double lr,
                        double beta1, double beta2, double eps, double weight_decay, int64_t step,
                        const int64_t* step_dev, double clip, double total_params);

/* dst(dtype_dst)[i] = src(dtype_src)[i]  (fp32 <-> bf16 conversion, round to nearest even). */
int rtp_cast(void* stream, int dtype_src, const void* src, int dtype_dst, void* dst, int64_t n);

/* ---------------------------------------------------------------------------------------------
 * Measurement (no counterpart in the reference, which only prints words/s:
 * benchmarks/rtp_benchmark.py:192-208).  With profiling enabled every kernel launch made by this
 * library is bracketed by two HIP timing events on the stream it is launched on and booked under
 * its kernel-variant name with the algorithmic flops and bytes of that launch.  rtp_profile_collect
 * synchronises the device, sums the event durations per name into `out` (at most `max_out`
 * entries, *n_out receives the count) and clears the records.  rtp_profile_read does the same without
 * clearing them.  Event timing (mode 1) is for eager launches only: timing events recorded while a stream is
 * captured into a HIP graph read 0 after a replay, so a launch made on a capturing stream is not timed in mode 1.
 * Launches inside a replayed graph are timed by mode 2 (below).
 * --------------------------------------------------------------------------------------------- */
typedef struct {
  char name[64];
  int64_t launches;
  double total_ms;
  double flops; /* algorithmic, summed over launches */
  double bytes; /* algorithmic, summed over launches */
  /* mode 2, wave-specialised product kernels only (else 0): where a workgroup's time goes, each entry the average over
   * every 16th workgroup of the launch, summed over launches: [0] launch start -> the workgroup's own start (waiting for a CU),
   * [1] its start -> first operands visible in LDS, [2] the K loop, [3] the epilogue */
  double phase_ms[4];
} rtp_kernel_stat;

int rtp_profile_enable(int mode); /* 0 off, 1 HIP events around every launch, 2 device time stamps (see below) */
/* Mode 2 is for launches recorded into a HIP graph, where timing events do not work: every rtp_gemm launch made
 * while it is on carries the address of a two-word slot in device memory, where its workgroups leave the earliest
 * start and the latest end of the device's constant-rate wall clock (and the per-workgroup phase sums behind
 * rtp_kernel_stat.phase_ms), at every replay.  rtp_profile_reset_stamps
 * (a small kernel on `stream`) clears the slots before a replay; rtp_profile_read after it returns that replay's
 * durations per kernel variant.  Other kernels are not timed in this mode. */
int rtp_profile_reset_stamps(void* stream);
int rtp_profile_collect(rtp_kernel_stat* out, int max_out, int* n_out);
int rtp_profile_read(rtp_kernel_stat* out, int max_out, int* n_out);

#ifdef __cplusplus
}
#endif
#endif /* RTP_HIP_H */
