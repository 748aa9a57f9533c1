/*
 * alpha_hip.h -- flat C ABI of libalpha_hip.so, the MI355X (gfx950) compute backend for the GPT
 * training step of alpha2.  This is the seam a Bun-FFI / N-API / ctypes shim binds; it replaces the
 * reference's only native seam, the N-API addon `helios_vk.c` (export table
 * packages/helios/native/helios_vk.c:4403-4432, typed in packages/helios/src/device.ts:17-39), and
 * provides one entry point per operation of the reference's `Backend` interface
 * (packages/core/src/interfaces.ts:38-151) that the training step reaches.
 *
 * Conventions
 *   - Every function returns int32 status, 0 = OK; ah_last_error() gives the message.  No C++
 *     exception crosses this boundary.  (Reference: napi_throw_error, helios_vk.c:3367,3405.)
 *   - Device memory is named by opaque uint64 handles that ARE device addresses; a handle plus a
 *     byte offset is a valid operand (views).  Only handles returned by ah_alloc may be freed.
 *   - Tensors are row-major contiguous unless a leading-dimension argument says otherwise.
 *   - One caller thread.  All work is enqueued on one persistent HIP stream in call order;
 *     ah_sync, ah_download, ah_download_end and ah_event_elapsed_ms are the only blocking calls.
 *   - dtype codes: AH_F32 activations/params/grads, AH_BF16 internal fast-mode storage,
 *     AH_I32 indices, AH_F16 storage-only cast target (the reference's Dtype has no bf16:
 *     packages/core/src/types.ts:6).
 */
#ifndef ALPHA_HIP_H
#define ALPHA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t ah_ptr;

enum { AH_F32 = 0, AH_BF16 = 1, AH_I32 = 2, AH_F16 = 3 };

enum {
  AH_OK = 0,
  AH_ERR_HIP = 1,        /* a HIP runtime call failed */
  AH_ERR_ARG = 2,        /* shape / dtype / alignment mismatch (reference: thrown Error, cpu_ref.ts:172-182) */
  AH_ERR_STATE = 3,      /* not initialised, or call illegal while a graph is being captured */
  AH_ERR_OOM = 4,
  AH_ERR_UNSUPPORTED = 5
};

/* ---- device / lifetime.  Replaces initDevice / destroy / waitIdle (helios_vk.c:4405-4425). ---- */
typedef struct {
  char     name[128];
  char     arch[32];          /* "gfx950..." */
  int32_t  compute_units;
  int32_t  wavefront;
  int32_t  clock_khz;
  int32_t  lds_bytes_per_block;
  uint64_t hbm_bytes;
} AhDeviceInfo;

int32_t     ah_init(int32_t device);
int32_t     ah_shutdown(void);
const char *ah_last_error(void);
int32_t     ah_device_info(AhDeviceInfo *out);
int32_t     ah_sync(void);

/* ---- buffers.  Replaces createBuffer / uploadBuffer / fillBuffer / readBuffer / destroyBuffer
 *      (helios_vk.c:4407-4412).  Frees are stream-ordered: a freed block is only ever reused by
 *      work enqueued later on the same stream. ---- */
int32_t ah_alloc(uint64_t bytes, ah_ptr *out);
int32_t ah_free(ah_ptr p);
int32_t ah_upload(ah_ptr dst, const void *host, uint64_t bytes);      /* host buffer borrowed for the call only */
int32_t ah_download(void *host, ah_ptr src, uint64_t bytes);          /* blocks until data has landed */
/* A read-back of at most 256 bytes in two halves, for a value that exists long before the host looks at it (the loss of a
 * step, which the reference's trainer reads after it has issued the whole backward pass, trainer.ts:1247): _begin queues the
 * copy into a pinned slot behind the work issued so far and returns a ticket; _end waits for THAT copy only - not for what
 * was issued after it - and hands the bytes over.  Sixteen tickets are held; an older one is refused (AH_ERR_STATE), and the
 * caller reads with ah_download instead.  Inside a step plan _begin is a boundary like ah_download; _end is none.  The
 * reference's counterpart is its lazy read-back against a timeline value (packages/helios/src/backend.ts:1143-1171,
 * helios_vk.c waitTimeline). */
int32_t ah_download_begin(ah_ptr src, uint64_t bytes, uint64_t *out_ticket);
int32_t ah_download_end(uint64_t ticket, void *host, uint64_t bytes);
int32_t ah_copy(ah_ptr dst, ah_ptr src, uint64_t bytes);              /* device to device */
int32_t ah_fill_f32(ah_ptr dst, float value, uint64_t n);
int32_t ah_fill_i32(ah_ptr dst, int32_t value, uint64_t n);

/* Counters the reference trainer polls through gpuMemStats()/gpuOpsThisStep/resetStepOps
 * (packages/train/src/trainer.ts:1003-1032,1821-1843,1915). */
typedef struct {
  uint64_t live_allocs;
  uint64_t live_bytes;
  uint64_t pool_blocks;
  uint64_t pool_bytes;
  uint64_t device_mallocs;      /* hipMalloc calls so far */
  uint64_t ops_launched;        /* kernels enqueued since ah_reset_op_count */
  uint64_t graphs_live;
  uint64_t steps_recorded;      /* ah_step_end results so far: plans recorded, steps replayed, steps that fell back */
  uint64_t steps_replayed;
  uint64_t steps_fallback;
  uint64_t step_node_updates;   /* kernel nodes whose arguments were rewritten during replays */
} AhStats;
int32_t ah_stats(AhStats *out);
int32_t ah_reset_op_count(void);
int32_t ah_trim_pool(void);      /* purgeBufferPools (trainer.ts:1012): return cached blocks to the driver */

/* ---- whole-step capture.  Replaces batchBegin / batchSubmit / batchExecuteAll
 *      (helios_vk.c:4414-4419): everything enqueued between begin and end becomes one hipGraph.
 *      Blocks allocated while capturing belong to the graph until ah_graph_destroy. ---- */
int32_t ah_graph_begin(void);
int32_t ah_graph_end(uint64_t *out_graph);
int32_t ah_graph_launch(uint64_t graph);
int32_t ah_graph_destroy(uint64_t graph);

/* ---- step plans: record -> verify -> replay.  The caller keeps issuing the SAME Backend-level calls every training step
 *      (the reference's tape-driven trainer, packages/train/src/trainer.ts:1188-1273,1761-1784, cannot do otherwise); the library
 *      turns them into graph launches.  Between ah_step_begin(key) and ah_step_end:
 *        - with no plan for `key`, every kernel launch is captured instead of run; at each point where the host needs the
 *          stream (ah_download, ah_sync, ...) the launches so far become one hipGraph segment, which is launched, and capture
 *          resumes.  ah_step_end stores the segments as the plan (result AH_STEP_RECORDED).
 *        - with a plan, every call is compared with the plan's next kernel node: same kernel and grid means the launch is
 *          skipped (the graph holds it); arguments that differ (learning rate, bias corrections, seeds, a buffer that moved)
 *          are written into the node.  Boundaries launch the segment's graph.  ah_upload copies into a pinned slot owned by
 *          the plan, read by a copy node.  Result AH_STEP_REPLAYED.
 *        - the first call that does not match (another kernel, another grid, a boundary elsewhere) ends the replay: the
 *          skipped launches of the open segment are issued from the plan, the rest of the step runs eagerly, the plan is
 *          dropped and the next step records again (AH_STEP_FELL_BACK; ah_step_note() says what differed).
 *      Results are those of eager execution in every case.  Replaces the reference's per-step batching of dispatches
 *      (batchBegin / batchDispatchMany / batchSubmit, helios_vk.c:4414-4419; packages/helios/src/backend.ts:880-1134). ---- */
/*      A bracket in which nothing was issued changes nothing (AH_STEP_EAGER). */
enum { AH_STEP_EAGER = 0, AH_STEP_RECORDED = 1, AH_STEP_REPLAYED = 2, AH_STEP_FELL_BACK = 3 };
int32_t     ah_step_begin(uint64_t key);
int32_t     ah_step_end(int32_t *out_how);
int32_t     ah_step_reset(uint64_t key);          /* drop the plan of `key` */
/* A hint from a caller that is about to spend host time before its next launches (e.g. between the first and the later
 * adamwStep calls of an optimizer pass, packages/train/src/optimizers.ts:54-94): what has been issued since the last boundary
 * becomes a segment of its own and is launched now instead of waiting for the segment to fill.  Part of the plan like any
 * other boundary (a replay expects it at the same place); a no-op outside a step and when nothing has been issued.  The
 * reference's counterpart is an early batchSubmit (helios_vk.c:4417). */
int32_t     ah_step_kick(void);
const char *ah_step_note(void);                    /* why the last step fell back ("" if it did not) */

/* ---- a side stream (same priority) for work nothing depends on for a while, e.g. weight gradients, which only the
 *      gradient norm reads: launches between ah_side_begin and ah_side_end go to the side stream, which first waits for
 *      everything issued on the main stream so far; the main stream carries on at once.  ah_side_join makes the main stream
 *      wait for all side work.  Legal inside ah_graph_begin .. ah_graph_end (the fork and join become graph edges; join
 *      before ah_graph_end) and a no-op inside a step plan.  Allocation and frees stay ordered on the main stream: buffers
 *      that side work reads or writes must not be freed before ah_side_join.  Only ah_gemm (without its split-K path),
 *      ah_gemm_grouped_run / _run_sumsq and ah_embedding_index may be issued between ah_side_begin and ah_side_end: the entry points that work
 *      through the library's one scratch buffer (the reductions, ah_layernorm_bwd, ah_cross_entropy*, ah_channel_act_bwd,
 *      the Adafactor steps) are refused there (AH_ERR_OOM, "no scratch"), and those that take a workspace
 *      from the pool (ah_embedding_bwd, the one-pass flash backward, split-K products) would have it handed back to the
 *      main stream while the side stream still uses it: do not issue them there.  No counterpart in the reference, whose
 *      dispatches are strictly serial (helios_vk.c:3291-3328 orders them with buffer barriers). ---- */
int32_t ah_side_begin(void);
int32_t ah_side_end(void);
int32_t ah_side_join(void);

/* ---- timing on the library stream.  Replaces gpuTime (helios_vk.c:3448). ---- */
int32_t ah_event_create(uint64_t *out_event);
int32_t ah_event_record(uint64_t event);
int32_t ah_event_elapsed_ms(uint64_t start, uint64_t stop, float *out_ms);   /* blocks on `stop` */
int32_t ah_event_destroy(uint64_t event);

/* ---- element-wise, f32.  Backend.add/sub/mul/div/neg/exp/log/sqrt/pow/scale/clamp/gelu/relu/silu
 *      (interfaces.ts:49-73; cpu_ref.ts:150-164,334-360,422-435). ---- */
enum { AH_ADD = 0, AH_SUB = 1, AH_MUL = 2, AH_DIV = 3 };
enum { AH_NEG = 0, AH_EXP = 1, AH_LOG = 2, AH_SQRT = 3, AH_POW = 4, AH_SCALE = 5, AH_CLAMP = 6,
       AH_GELU = 7, AH_RELU = 8, AH_SILU = 9, AH_SOFTCAP = 10 };
/* same-shape binary */
int32_t ah_binary(int32_t op, ah_ptr a, ah_ptr b, ah_ptr out, uint64_t n);
/* NumPy-broadcast binary: out has `nd` dims `shape`; a/b element strides per dim (0 = broadcast)
 * (packages/core/src/broadcast.ts:13-65). nd <= 6. */
int32_t ah_binary_broadcast(int32_t op, ah_ptr a, ah_ptr b, ah_ptr out, int32_t nd,
                            const int64_t *shape, const int64_t *stride_a, const int64_t *stride_b);
int32_t ah_unary(int32_t op, ah_ptr x, ah_ptr out, uint64_t n, float p0, float p1);
/* in place: Backend.addInplace / scaleInplace (interfaces.ts:113-114) */
int32_t ah_add_inplace(ah_ptr a, ah_ptr b, uint64_t n);
int32_t ah_scale_inplace(ah_ptr a, float s, uint64_t n);
/* out = a + b on bf16 storage, rounded once (Backend.add / addInplace, interfaces.ts:49,113, for tensors a bf16 backend keeps
 * in bf16: the tape's gradient accumulation, tape.ts:116-127); out may be a or b; 16-byte aligned */
int32_t ah_add_bf16(ah_ptr a, ah_ptr b, ah_ptr out, uint64_t n);
/* a[i] += b[i] * s  -- loss accumulation over micro-steps (trainer.ts:1208-1223) without a temporary */
int32_t ah_axpy_inplace(ah_ptr a, ah_ptr b, float s, uint64_t n);

/* backward element-wise: Backend.geluBackward/reluBackward/siluBackward/clampBackward/
 * softCapBackward/siluMul/siluMulBackward (interfaces.ts:96-106; CPU fallbacks ops.ts:284-417) */
enum { AH_GELU_BWD = 0, AH_RELU_BWD = 1, AH_SILU_BWD = 2, AH_CLAMP_BWD = 3, AH_SOFTCAP_BWD = 4 };
int32_t ah_unary_bwd(int32_t op, ah_ptr x, ah_ptr grad_out, ah_ptr out, uint64_t n, float p0, float p1);
int32_t ah_silu_mul(ah_ptr a, ah_ptr b, ah_ptr out, uint64_t n);
int32_t ah_silu_mul_bwd(ah_ptr a, ah_ptr b, ah_ptr grad_out, ah_ptr da, ah_ptr db, uint64_t n);
/* Per-channel mixture of activation bases, the MLP activations "universal" (silu(h)*gate + h*skip) and "kan_spline"
 * (c0 silu + c1 relu + c2 gelu + c3 h + c4 h^2) that the reference composes from separate ops (packages/model/src/gpt.ts:295-321),
 * in one pass:  out[r,c] = sum_k coefs[k][c] * basis_k(x[r,c])  over the bases whose bit is set in `mask`
 * (bit 0 silu, 1 relu, 2 tanh-gelu, 3 identity, 4 square).  dtype (AH_F32 or AH_BF16) is the type of x, out, grad_out and dx;
 * coefs: 5 handles of f32[cols]; a 0 handle (or coefs == NULL) for a selected basis is the constant 1, so one selected basis
 * without coefficients is the plain silu / relu / gelu MLP activation.  cols % 4 == 0.
 * Backward: dx = grad_out * sum_k coefs[k] * basis_k'(x);  dcoefs[k][c] = sum_r grad_out[r,c] * basis_k(x[r,c]) for the bases
 * that have a coefficient vector (column sums in fixed order; overwritten, or added to when `accumulate` is non-zero:
 * gradient accumulation over micro-steps, trainer.ts:1164-1273). */
int32_t ah_channel_act(int32_t dtype, ah_ptr x, const ah_ptr *coefs, int32_t mask, ah_ptr out, int64_t rows, int64_t cols);
int32_t ah_channel_act_bwd(int32_t dtype, ah_ptr x, const ah_ptr *coefs, int32_t mask, ah_ptr grad_out, ah_ptr dx, const ah_ptr *dcoefs,
                           int32_t accumulate, int64_t rows, int64_t cols);
/* SwiGLU on a packed pre-activation (packages/model/src/gpt.ts:295-299 computes silu(x Wgate^T) * (x Wup^T) with
 * Backend.siluMul, interfaces.ts:105-106): gate_up = [rows, 2 cols], gate in the first `cols` columns of a row and up in
 * the last -- what ONE product with the two weight matrices stacked gives.  out[r,c] = silu(gate[r,c]) * up[r,c];
 * backward writes d_gate_up in the same packed layout.  dtype AH_F32 or AH_BF16 for every operand; cols % 4 == 0. */
int32_t ah_swiglu(int32_t dtype, ah_ptr gate_up, ah_ptr out, int64_t rows, int64_t cols);
int32_t ah_swiglu_bwd(int32_t dtype, ah_ptr gate_up, ah_ptr grad_out, ah_ptr d_gate_up, int64_t rows, int64_t cols);
/* Backend.residualDropoutAdd: out = residual + projected*mask (interfaces.ts:110; mask may be 0 = no dropout) */
int32_t ah_residual_dropout_add(ah_ptr residual, ah_ptr projected, ah_ptr mask, ah_ptr out, uint64_t n);
/* Backend.dropoutMask (interfaces.ts:125): out[i] = hash(seed, counter, i) / 2^32 > p ? (float)(1/(1-p)) : 0 with the hash of the
 * reference's CPU path, DropoutRng.hash (packages/autograd/src/ops.ts:74-81), reproduced bit for bit for every index: its
 * first line is evaluated in doubles before the cut to 32 bits.  n <= 2^32. */
int32_t ah_dropout_mask(ah_ptr out, uint64_t n, int32_t seed, int32_t counter, double p);
/* Backend.residualDropoutAdd and the mask multiply of its backward (ops.ts:616-686) with the mask of ah_dropout_mask made on
 * the fly instead of stored: out[i] = (residual ? residual[i] : 0) + x[i] * mask(seed, counter, p)[i].  The seed is read from
 * device memory (one int32) when the kernel runs, so a captured step draws new masks at every replay: the host writes the
 * step's seed there before it launches the step (trainer.ts:1169,1202: seed + 1000 step + micro-step; counter = the mask's
 * place in the forward pass, ops.ts:25-82).  x is f32 or bf16; residual and out share out_dtype (f32 or bf16). */
int32_t ah_dropout_apply(ah_ptr x, int32_t x_dtype, ah_ptr residual, ah_ptr out, int32_t out_dtype, uint64_t n, ah_ptr seed_i32,
                         int32_t counter, double p);
/* Backend.maskedFill with the mask tiled by i % mask_n (cpu_ref.ts:891-911) */
int32_t ah_masked_fill(ah_ptr a, ah_ptr mask, ah_ptr out, uint64_t n, uint64_t mask_n, float value);
/* Backend.causalMask (cpu_ref.ts:880-889) */
int32_t ah_causal_mask(ah_ptr out, int64_t size);
/* Backend.castDtype f32<->f16 storage cast (interfaces.ts:139) and the internal f32<->bf16 cast */
int32_t ah_cast(ah_ptr src, int32_t src_dtype, ah_ptr dst, int32_t dst_dtype, uint64_t n);
/* Backend.checkFinite -> one f32: 0.0 all finite, 1.0 otherwise (interfaces.ts:146) */
int32_t ah_check_finite(ah_ptr x, uint64_t n, ah_ptr out_flag);

/* ---- data movement, 4-byte elements.  Backend.transpose/slice/scatterSlice/cat/sliceQkv/broadcast
 *      (cpu_ref.ts:578-694; interfaces.ts:117-136). nd <= 6. ---- */
int32_t ah_transpose(ah_ptr a, ah_ptr out, int32_t nd, const int64_t *shape, int32_t dim0, int32_t dim1);
int32_t ah_slice(ah_ptr a, ah_ptr out, int32_t nd, const int64_t *shape, const int64_t *starts, const int64_t *ends);
/* zero-fills `out` (orig_shape) and places grad at [starts, starts+gshape) */
int32_t ah_scatter_slice(ah_ptr grad, ah_ptr out, int32_t nd, const int64_t *gshape, const int64_t *orig_shape,
                         const int64_t *starts);
/* copies `src` (src_shape) into `dst` (dst_shape) at offset `axis_offset` along `axis` -- one call per cat() operand */
int32_t ah_cat_part(ah_ptr src, ah_ptr dst, int32_t nd, const int64_t *src_shape, const int64_t *dst_shape,
                    int32_t axis, int64_t axis_offset);
int32_t ah_slice_qkv(ah_ptr qkv, ah_ptr q, ah_ptr k, ah_ptr v, int64_t rows, int64_t d);
int32_t ah_broadcast(ah_ptr a, ah_ptr out, int32_t nd, const int64_t *out_shape, const int64_t *stride_a);

/* ---- reductions, f32.  Backend.sum/mean/softmax/logSoftmax/argmax (cpu_ref.ts:260-330,437-541,
 *      698-756), sumOfSquares/totalSumOfSquares (interfaces.ts:144-145). The tensor is viewed as
 *      [outer, dim, inner] with the reduced axis in the middle. ---- */
int32_t ah_sum_axis(ah_ptr a, ah_ptr out, int64_t outer, int64_t dim, int64_t inner, int32_t mean);
int32_t ah_sum_all(ah_ptr a, ah_ptr out, uint64_t n, int32_t mean);
int32_t ah_softmax(ah_ptr a, ah_ptr out, int64_t outer, int64_t dim, int64_t inner, int32_t log_softmax);
/* first maximum wins, NaN never selected, i32 result: bit-exact with cpu_ref.ts:698-756 */
int32_t ah_argmax(ah_ptr a, ah_ptr out_i32, int64_t outer, int64_t dim, int64_t inner);
/* out[0] (f32) = sum of x^2 over n elements; deterministic two-stage f64 reduction */
int32_t ah_sum_sq(ah_ptr x, uint64_t n, ah_ptr out);
/* The same over a list of tensors as ONE number: Backend.totalSumOfSquares (interfaces.ts:145), which the trainer calls on
 * the whole gradient set (trainer.ts:1345-1349).  One launch per 120 tensors plus one for the final sum, instead of three per
 * tensor; the partition into partial sums (chunks of 16384 elements per tensor) depends on the sizes only. */
int32_t ah_sum_sq_list(const ah_ptr *xs, const uint64_t *ns, int32_t count, ah_ptr out);
/* ah_sum_sq for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): it has no counterpart in the reference.  Same kernels, same partition and so bit-identical results, but the
 * partial sums live in a 32 KiB array that is part of the library image on each device (held until the process ends) instead
 * of pool scratch; the call makes no hipMalloc / hipFree and no allocating library call.  1 <= n <= 2^32 elements, anything
 * larger is refused with AH_ERR_ARG.  All calls on one GPU share that array: calls that overlap on one GPU (other streams,
 * other threads) race; calls on this library's single stream are ordered and safe. */
int32_t ah_sum_sq_static(ah_ptr x, uint64_t n, ah_ptr out);
/* softmax backward: s*(g - sum(g*s)) over the last dim (ops.ts:688-700), rows x dim */
int32_t ah_softmax_bwd(ah_ptr s, ah_ptr g, ah_ptr out, int64_t rows, int64_t dim);

/* ---- nn.  Backend.embedding / embeddingBackward (cpu_ref.ts:364-385; ops.ts:491-507),
 *      layerNorm / layerNormBackward (cpu_ref.ts:387-420; ops.ts:509-571),
 *      crossEntropy / crossEntropyBackward (cpu_ref.ts:543-563; ops.ts:702-729). ---- */
/* out[i] = weight[idx[i]]; an id outside [0, vocab) gives a row of NaN, which is what the reference's loop stores when it
 * reads past the weight array (cpu_ref.ts:364-385), and no access outside the array is made. */
int32_t ah_embedding(ah_ptr weight, ah_ptr idx_i32, ah_ptr out, int64_t n_idx, int64_t dim, int64_t vocab,
                     int32_t out_dtype);
/* out[i] = wte[tok[i]] + wpe[i % T]  -- tok+pos embedding and the add of gpt.ts:362-379 in one pass */
int32_t ah_embedding_tok_pos(ah_ptr wte, ah_ptr wpe, ah_ptr tok_i32, ah_ptr out, int64_t n_idx, int64_t T,
                             int64_t dim, int64_t vocab, int32_t out_dtype);
/* grad_w[vocab,dim] = scatter-add of grad_out rows (zero-filled first unless accumulate != 0); ids outside [0, vocab) are
 * skipped.  Up to 32768 positions over fewer than 65535 ids (rows of 4 k floats) the order of the additions is fixed: the
 * positions are sorted by (id, position), the rows of an id are added in position order inside chunks of 32 sorted positions
 * (as the reference's loop adds them, packages/autograd/src/ops.ts:491-507) and the chunks of a longer run in chunk order, so
 * the result is the same from run to run.  Beyond those sizes the rows are added with f32 atomics (order not fixed). */
int32_t ah_embedding_bwd(ah_ptr idx_i32, ah_ptr grad_out, ah_ptr grad_w, int64_t n_idx, int64_t dim,
                         int64_t vocab, int32_t accumulate);
/* The same in two steps for a token batch that stays on the device for several backward passes (a resident batch, the
 * micro-batches of an accumulating step): ah_embedding_index sorts once into `index_out` (ah_embedding_index_bytes(n_idx, vocab)
 * bytes; 0 = sizes outside the fixed-order path), ah_embedding_bwd_indexed is ah_embedding_bwd without the sort. */
int64_t ah_embedding_index_bytes(int64_t n_idx, int64_t vocab);
int32_t ah_embedding_index(ah_ptr idx_i32, int64_t n_idx, int64_t vocab, ah_ptr index_out);
int32_t ah_embedding_bwd_indexed(ah_ptr index, ah_ptr grad_out, ah_ptr grad_w, int64_t n_idx, int64_t dim, int64_t vocab,
                                 int32_t accumulate);
/* grad_wpe[T,dim] (+)= sum over the batch of grad_out[b,t,:]  (positions are 0..T-1 per row) */
int32_t ah_pos_embedding_bwd(ah_ptr grad_out, ah_ptr grad_wpe, int64_t batch, int64_t T, int64_t dim,
                             int32_t accumulate);
/* Batch assembly of DataLoader.nextBatch (packages/train/src/data.ts:94-167) from a corpus resident on the device:
 *   inputs[b,t] = corpus[(start[b] + t) mod n_tokens],  targets[b,t] = corpus[(start[b] + t + 1) mod n_tokens].
 * Random mode never wraps (start < n_tokens - T); packed mode wraps exactly as the reference's cursor loop does
 * (the target of the corpus' last token is its first).  corpus, inputs, targets: i32; starts: i64[batch] on the device. */
int32_t ah_token_windows(ah_ptr corpus_i32, int64_t n_tokens, ah_ptr starts_i64, int64_t batch, int64_t T,
                         ah_ptr inputs_i32, ah_ptr targets_i32);
/* x_dtype: AH_F32, or AH_BF16 (with a bf16 result) for a caller that keeps its residual stream in bf16 */
int32_t ah_layernorm(ah_ptr x, ah_ptr w, ah_ptr b, ah_ptr out, int64_t rows, int64_t dim, float eps,
                     int32_t out_dtype, int32_t x_dtype);
/* dx (+= residual_grad when that handle is non-zero), dw, db.  dw/db are deterministic column sums;
 * accumulate != 0 adds them into existing dw/db (gradient accumulation). grad_out dtype f32 or bf16.
 * dx_bf16 (0 = none) also receives dx rounded to bf16, the operand of the next backward GEMMs.
 * stream_dtype = the type of x and residual_grad: AH_F32, or AH_BF16 for a residual stream kept in bf16 (then grad_out is
 * bf16, dim % 4 == 0, dim <= 2048, dx_bf16 is required and dx may be 0). */
int32_t ah_layernorm_bwd(ah_ptr x, ah_ptr w, ah_ptr grad_out, int32_t grad_dtype, ah_ptr residual_grad,
                         ah_ptr dx, ah_ptr dx_bf16, ah_ptr dw, ah_ptr db, int64_t rows, int64_t dim, float eps,
                         int32_t accumulate, int32_t stream_dtype);
/* The same with the column sums put off: the per-block partial sums of dw and db go to `partials` (caller-owned, at
 * least ah_layernorm_bwd_partials_bytes(rows, dim) bytes, which is 0 before ah_init), and ONE later call of
 * ah_layernorm_colsums reduces those of many LayerNorms (the 2 L + 1 of a model's backward pass) in one launch instead of
 * one small launch each; per job the result is bit-identical to ah_layernorm_bwd's.  The reference computes dw / db inside
 * layerNormBackward (packages/tensor/src/cpu_ref.ts, layerNormBackward); nothing of this split shows at the Backend level.
 * stream_dtype = the type of x and residual_grad: AH_F32, or AH_BF16 for a residual stream and gradient stream kept in bf16
 * (bf16 grad_out, dim % 4 == 0, dim <= 2048); dx (f32) may then be 0, dx_bf16 being the stream that the next call adds to. */
typedef struct {
  ah_ptr  partials, dw, db;
  int64_t rows, dim;          /* as passed to ah_layernorm_bwd_deferred */
  int32_t accumulate, reserved;
} AhColsumJob;
int64_t ah_layernorm_bwd_partials_bytes(int64_t rows, int64_t dim);
int32_t ah_layernorm_bwd_deferred(ah_ptr x, ah_ptr w, ah_ptr grad_out, int32_t grad_dtype, ah_ptr residual_grad,
                                  ah_ptr dx, ah_ptr dx_bf16, ah_ptr partials, int64_t rows, int64_t dim, float eps,
                                  int32_t stream_dtype);
int32_t ah_layernorm_colsums(const AhColsumJob *jobs, int32_t count);
/* loss[0] = mean_i (logsumexp(logits[i,:]) - logits[i,target[i]]); lse[N] kept for backward (0 = skip) */
int32_t ah_cross_entropy(ah_ptr logits, int32_t logits_dtype, ah_ptr targets_i32, ah_ptr loss_out, ah_ptr lse_out,
                         int64_t n, int64_t c);
/* dlogits = (softmax - onehot) * g[0] * g_mul / N; g_scalar = device f32 (0 = use 1.0); may run in place */
int32_t ah_cross_entropy_bwd(ah_ptr logits, int32_t dtype, ah_ptr targets_i32, ah_ptr lse, ah_ptr g_scalar,
                             float g_mul, ah_ptr dlogits, int64_t n, int64_t c);
/* Both of the above in one launch (crossEntropy + crossEntropyBackward, interfaces.ts:74,104; the backward of the loss
 * does not depend on its value): bf16 rows of up to 51200 classes are read ONCE, kept in registers between the two
 * halves, and the results are bit-identical to the pair; anything else runs the pair.  May run in place. */
int32_t ah_cross_entropy_fwd_bwd(ah_ptr logits, int32_t dtype, ah_ptr targets_i32, ah_ptr loss_out, ah_ptr lse_out,
                                 ah_ptr g_scalar, float g_mul, ah_ptr dlogits, int64_t n, int64_t c);

/* ---- GEMM on MFMA.  Backend.matmul / matmulTransposed / matmulTransposedA (cpu_ref.ts:166-258;
 *      interfaces.ts:111-112; autograd use ops.ts:197-234).  C[M,N] = op(A) * op(B):
 *        AH_GEMM_NN: A[M,K] * B[K,N]      (matmul;            dX = G * W)
 *        AH_GEMM_NT: A[M,K] * B[N,K]^T    (matmulTransposed;  Y = X * W^T)
 *        AH_GEMM_TN: A[K,M]^T * B[K,N]    (matmulTransposedA; dW = G^T * X)
 *      f32 operands -> fp32 MFMA (parity mode); bf16 operands -> bf16 MFMA with fp32 accumulation.
 *      lda/ldb/ldc are row strides in elements.  batch > 1 repeats with the given element strides
 *      (0 = operand shared across the batch).
 *      Epilogues: AH_EPI_NONE; AH_EPI_ACCUM  C += acc (gradient accumulation);
 *      AH_EPI_GELU  C = gelu(acc), aux (same dtype/ld as C) = acc  (matmulTransposedGelu, ops.ts:426-487);
 *      AH_EPI_RESIDUAL  C = acc + aux (aux [M,N] of C's dtype, ld = ldc; f32, or bf16 from bf16 operands) (residual add of gpt.ts:280-281);
 *      AH_EPI_GELU_BWD  C = acc * gelu'(aux) (aux = saved pre-activation, dtype of C);
 *      AH_EPI_GELU_GRAD C = gelu(acc), aux = gelu'(acc): the forward saves the derivative instead of the pre-activation,
 *      so that the backward product needs only  AH_EPI_MUL_AUX  C = acc * aux  (one multiply per element instead of
 *      re-evaluating the tanh; same mathematics as GELU / GELU_BWD with gelu' rounded to the storage type).
 *      Provided combinations: NONE -> f32 or bf16 output; ACCUM and RESIDUAL -> f32 output; GELU, GELU_BWD,
 *      GELU_GRAD and MUL_AUX -> output of the operand type.  Anything else returns AH_ERR_UNSUPPORTED. ---- */
enum { AH_GEMM_NN = 0, AH_GEMM_NT = 1, AH_GEMM_TN = 2 };
enum { AH_EPI_NONE = 0, AH_EPI_ACCUM = 1, AH_EPI_GELU = 2, AH_EPI_RESIDUAL = 3, AH_EPI_GELU_BWD = 4, AH_EPI_GELU_GRAD = 5, AH_EPI_MUL_AUX = 6 };
typedef struct {
  int32_t layout;            /* AH_GEMM_* */
  int32_t in_dtype;          /* AH_F32 or AH_BF16 (both operands) */
  int32_t out_dtype;         /* AH_F32 or AH_BF16 */
  int32_t epilogue;          /* AH_EPI_* */
  int64_t m, n, k;
  int64_t lda, ldb, ldc;
  int64_t batch;
  int64_t stride_a, stride_b, stride_c;
  ah_ptr  a, b, c, aux;
} AhGemm;
int32_t ah_gemm(const AhGemm *g);
/* ah_gemm with one operand in planes, so that a fused projection needs no copy around it.  Replaces the data movement of
 * Backend.sliceQkv (interfaces.ts:117; ops.ts:816-840: the [rows, 3C] product cut into three contiguous [rows, C]
 * tensors) and of the three Backend.scatterSlice results added up in its backward (interfaces.ts:121; ops.ts:826-834):
 *   c_plane_cols > 0: columns [p c_plane_cols, (p + 1) c_plane_cols) of C are stored as the [m, c_plane_cols] matrix at
 *     c + p * c_plane_stride (elements) with row stride ldc: the product writes q, k and v where sliceQkv would put them;
 *   a_plane_k > 0: columns [p a_plane_k, (p + 1) a_plane_k) of the row-major A [m, k] are read from the [m, a_plane_k] matrix
 *     at a + p * a_plane_stride with row stride lda (1 to 3 planes): the product reads dq, dk, dv where flash attention's
 *     backward leaves them, as if scattered into one [rows, 3C] gradient and added.
 * One plain product (layout NN or NT, bf16 operands and result, batch 1) on the 256-row tile kernel: m >= 256, n >= 128,
 * k and a_plane_k % 64 == 0, c_plane_cols % 128 == 0, operands 16-byte aligned with lda, ldb % 8 == 0; anything else returns
 * AH_ERR_UNSUPPORTED and the caller moves the data instead.  dry_run != 0 only answers (AH_OK / AH_ERR_UNSUPPORTED), nothing is launched. */
int32_t ah_gemm_planes(const AhGemm *g, int64_t c_plane_cols, int64_t c_plane_stride, int64_t a_plane_k, int64_t a_plane_stride,
                       int32_t dry_run);
/* Grouped GEMM: several independent problems of ONE layout in one launch (256x256 tiles of all problems share the
 * grid, so small outputs with a long contraction fill the chip without split-K).  Used for the weight gradients
 * dW_i = G_i^T X_i of all layers at the end of backward; the reference computes them one matmul at a time
 * (packages/autograd/src/ops.ts:197-234).  Requirements per problem: bf16 operands, batch 1, k a multiple of 64,
 * 16-byte aligned rows, epilogue NONE or ACCUM; all problems share layout and output type.  The plan copies the
 * descriptors to the device once; ah_gemm_grouped_run only launches (safe inside graph capture) and takes the
 * epilogue (AH_EPI_NONE, or AH_EPI_ACCUM for f32 outputs) so one plan serves first and later micro-batches.
 * Tiles run one per CU in rounds of 256; when the last round of an f32 plan is at most half full, the plan cuts the
 * problems that make up that round in two along k (second halves into a workspace the plan owns, added to C by a short
 * second kernel in a fixed order), which halves the cost of that round; ah_gemm_last_kernel then reports 2 slices. */
int32_t ah_gemm_grouped_plan(const AhGemm *descs, int32_t count, uint64_t *plan_out);
int32_t ah_gemm_grouped_run(uint64_t plan, int32_t epilogue);
/* ah_gemm_grouped_run of an f32 plan that also adds, to the f32 at sumsq_inout, the sum of the squares of every value the
 * run leaves in the C matrices (after ACCUM: of the accumulated values): the weight gradients' share of the norm that
 * Backend.totalSumOfSquares (interfaces.ts:145; trainer.ts:1345-1349) computes by reading every gradient again.  The
 * squares are taken in the epilogue, from the registers that are being stored, summed per wave in f32 and over the waves
 * in f64 in an order that depends on the plan only (same result from run to run).  Four floats per 256 x 256 tile of
 * scratch, which the plan owns. */
int32_t ah_gemm_grouped_run_sumsq(uint64_t plan, int32_t epilogue, ah_ptr sumsq_inout);
/* The same problems at other addresses (a caller whose gradient buffers are new tensors every step: the tape's weight
 * gradients, packages/autograd/src/ops.ts:197-234): rewrites the plan's device tables from a descriptor list with the shapes
 * the plan was made for, without allocating.  Two small uploads; a list of other shapes is refused. */
int32_t ah_gemm_grouped_update(uint64_t plan, const AhGemm *descs, int32_t count);
int32_t ah_gemm_grouped_destroy(uint64_t plan);
/* Profiling aid (no counterpart in the reference): writes the name of the kernel the most recent ah_gemm call
 * launched, spelled as a profiler demangles it (e.g. "k_gemm_bf16<256, 256, 2, 4, false, false>"), and the number
 * of split-K slices it used (1 = none; > 1 means a k_splitk_reduce launch followed). */
int32_t ah_gemm_last_kernel(char *name, int32_t capacity, int32_t *nsplit);
/* Measurement aid (no counterpart in the reference; the nearest is the flop accounting of scripts/bench-ops.ts:302-328, which
 * prices GEMMs against a peak): ONE launch in which every SIMD of the device runs waves_per_simd (1-4) waves that each issue
 * iters (1-200000) x 8 independent 32x32x16 bf16 MFMAs on operands held in registers: no LDS, no memory traffic.
 * random_operands != 0: operands of the size of activations and weights with pseudo-random bits; 0: all zeros.  *flops_out (host,
 * may be null) = the flops of the launch.  Timed by the caller with ah_event_*: with zeros the part runs at its published
 * dense peak, with operands whose bits toggle at what its power limit sustains, which is the ceiling a GEMM on real data
 * can be read against. */
int32_t ah_probe_mfma_bf16(int32_t waves_per_simd, int32_t iters, int32_t random_operands, double *flops_out);
/* Measurement aid (no counterpart in the reference): ONE launch in which every SIMD of the device runs waves_per_simd waves that
 * each issue iters (1-200000) x 32 groups of instructions on registers (no memory traffic).  kind 0: a group is one v_fma_f32;
 * 1: one v_exp_f32; 2: one v_exp_f32 and three v_fma_f32; 3: one 32x32x16 bf16 MFMA; 4 / 5: that MFMA followed by 8 / 16
 * v_fma_f32.  waves_per_simd 1-4 (1-2 with an MFMA in the group).  *groups_per_simd_out (host, may be null) = groups issued on
 * each SIMD.  Timed by the caller with ah_event_*: the time per group says what one wave alone can issue, what several waves
 * issue together, and how much of the vector work fits beside an MFMA -- the figures the attention kernels, which are bound
 * by per-score vector instructions, are read against. */
int32_t ah_probe_issue(int32_t kind, int32_t waves_per_simd, int32_t iters, double *groups_per_simd_out);

/* ---- fused causal flash attention.  Backend.flashAttention / flashAttentionBackward
 *      (interfaces.ts:127-135; kernel semantics packages/helios/src/kernels/attention.ts:1-586):
 *      s = (q.k)*scale; s = cap*tanh(s/cap) if cap > 0; keys after the query masked; online softmax;
 *      O = P V; LSE = m + log(l).  Element (b, h, t, d) of Q lives at q + b*q_sb + h*q_sh + t*q_st + d
 *      (same strides for K, V; o_* for O and dO; dq/dk/dv use the q strides), so both the reference's
 *      [B*H, T, D] contract and a [B*T, 3C] QKV projection read in place are expressible.
 *      LSE is [B, H, T] f32.  head_dim: a multiple of 8 from 8 to 128 (the kernels are built for 32, 64 and 128; another size
 *      runs the next larger one with the missing features read as zeros and never stored). ---- */
typedef struct {
  int32_t dtype;             /* AH_F32 (fp32 MFMA) or AH_BF16 */
  int32_t batch, heads, seq, head_dim;
  int64_t q_sb, q_sh, q_st;
  int64_t k_sb, k_sh, k_st;
  int64_t v_sb, v_sh, v_st;
  int64_t o_sb, o_sh, o_st;
  float   scale, soft_cap;
  ah_ptr  q, k, v, o, lse;
  ah_ptr  d_o, dq, dk, dv;   /* backward only; dq/dk/dv share the strides of q/k/v */
  int32_t bwd_variant;       /* backward, bf16, head_dim <= 64: 0 = a dQ kernel and a dK/dV kernel (each evaluates every score);
                                1 = one pass over the scores (a workgroup per 256 keys, dQ parts reduced in a fixed order).
                                Same results to bf16 rounding, both deterministic; 0 is the faster one today. */
  int32_t reserved;
} AhFlash;
int32_t ah_flash_fwd(const AhFlash *f);
int32_t ah_flash_bwd(const AhFlash *f);

/* ---- optimizer.  Backend.adamwStep (interfaces.ts:149-150; CPU loop optimizers.ts:76-92). ---- */
typedef struct {
  float lr, beta1, beta2, eps, weight_decay, bc1, bc2, grad_scale;
} AhAdamW;
/* In place on p, m, v (f32).  `dev_scale` (0 or a device f32) multiplies grad_scale on the device, so a
 * clip coefficient computed by ah_clip_coef never visits the host.  `dev_hyper` (0 or a device AhAdamW)
 * overrides `h` with values read on the device: a captured graph then follows per-step lr / bias
 * corrections written by ah_upload between launches.  `bf16_shadow` (0 or bf16[n]) receives the updated
 * parameters rounded to bf16 for the next step's MFMA operands.  When the effective gradient scale
 * (grad_scale x dev_scale[0]) is not finite the call changes nothing (see ah_step_guard). */
int32_t ah_adamw(ah_ptr p, ah_ptr g, ah_ptr m, ah_ptr v, uint64_t n, const AhAdamW *h, ah_ptr dev_hyper,
                 ah_ptr dev_scale, ah_ptr bf16_shadow);
/* The same update for a list of tensors in one launch per 48 of them: what AdamW.stepParamEntries (optimizers.ts:54-94) does
 * tensor by tensor.  h, dev_hyper and dev_scale as for ah_adamw; the weight decay is per item (the no-decay set). */
typedef struct { ah_ptr p, g, m, v, shadow; uint64_t n; float weight_decay; int32_t reserved; } AhAdamWItem;
int32_t ah_adamw_list(const AhAdamWItem *items, int32_t count, const AhAdamW *h, ah_ptr dev_hyper, ah_ptr dev_scale);
/* out[0] = clip / (sqrt(sumsq[0]) * |grad_scale|) if that norm exceeds clip, else 1  (trainer.ts:1650-1656);
 * out[1] = the norm itself. */
int32_t ah_clip_coef(ah_ptr sumsq, float grad_scale, float clip, ah_ptr out2);
/* The same for a step that never visits the host, together with what the reference trainer decides there between backward and
 * the optimizer call: a loss (0 = not checked) or gradient norm that is not finite skips the step (trainer.ts:1248-1262,
 * 1495-1522).  out[0] = clip coefficient, or NaN to skip -- ah_adamw leaves p, m, v and the shadow untouched when its effective
 * gradient scale is not finite; out[1] = the norm; out[2] = 1 if skipped else 0.  state = 3 doubles on the device
 * {beta1^t, beta2^t, steps skipped}: on an applied step the powers advance and bc1 = 1 - beta1^t, bc2 = 1 - beta2^t are written
 * into the device AhAdamW `dev_hyper` (optimizers.ts:107-115 advances them only when the optimizer runs); on a skipped step
 * nothing but the skip count changes. */
int32_t ah_step_guard(ah_ptr sumsq, ah_ptr loss, float grad_scale, float clip, double beta1, double beta2, ah_ptr state_f64x3,
                      ah_ptr dev_hyper, ah_ptr out3);

/* ---- the other optimizers of the reference's registry (optimizers.ts:596-603).  The reference runs them as host loops
 *      over Float32Arrays, i.e. in double precision with one rounding per store; the kernels compute in double the
 *      same way, so Lion and SGD reproduce the loops bit for bit and Adafactor up to the order of its double sums. ---- */
typedef struct { double lr, beta1, beta2, weight_decay, grad_scale; } AhLion;
/* Lion.stepTensor (optimizers.ts:284-311): in place on p and the momentum m (f32). */
int32_t ah_lion(ah_ptr p, ah_ptr g, ah_ptr m, uint64_t n, const AhLion *h);
/* SGD (optimizers.ts:555-567): p -= lr * (g * grad_scale). */
int32_t ah_sgd(ah_ptr p, ah_ptr g, uint64_t n, double lr, double grad_scale);
typedef struct { double lr, beta2, eps, clip_threshold, weight_decay, grad_scale; } AhAdafactor;
/* Adafactor.stepTensor, factored branch for a [rows, cols] parameter (optimizers.ts:412-475): vr f32[rows] and
 * vc f32[cols] are the row / column second moments, updated in place. */
int32_t ah_adafactor_2d(ah_ptr p, ah_ptr g, ah_ptr vr, ah_ptr vc, int64_t rows, int64_t cols, const AhAdafactor *h);
/* Adafactor.stepTensor, unfactored branch for any other parameter (optimizers.ts:478-500): v f32[n]. */
int32_t ah_adafactor_flat(ah_ptr p, ah_ptr g, ah_ptr v, uint64_t n, const AhAdafactor *h);

/* ---- host-side SeededRng (packages/core/src/rng.ts:6-68): int32 xorshift pair, 20 warm-up draws,
 *      next() = ((s0+s1)>>>0)/2^32, polar Box-Muller with a cached spare.  Pure host code (no device work);
 *      here so that parameter initialisation (packages/model/src/gpt.ts:53-59,73-151) draws the reference's
 *      stream at native speed. ---- */
typedef struct { int32_t s0, s1; int32_t has_spare; int32_t _pad; double spare; } AhRng;
int32_t ah_rng_seed(AhRng *r, int32_t seed);
int32_t ah_rng_next(AhRng *r, double *out);
int32_t ah_rng_next_gauss(AhRng *r, double *out);
int32_t ah_rng_fill_gauss_f32(AhRng *r, float *out, uint64_t n, double std);   /* out[i] = (float)(nextGauss()*std) */
int32_t ah_rng_fill_uniform_f64(AhRng *r, double *out, uint64_t n);

#ifdef __cplusplus
}
#endif
#endif /* ALPHA_HIP_H */
