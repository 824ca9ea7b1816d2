/*
 * tspipe_amd.h -- C ABI of the MI355X (gfx950) teacher-student step kernels.
 *
 * The reference (kaist-ina/TSPipe) has no native code and no FFI: every
 * operation below is, there, a chain of eager PyTorch calls made from a Python
 * plug-in.  Each entry point cites the reference lines whose arithmetic it
 * replaces; the Python adapters in tspipe_amd/ keep the reference's plug-in
 * signatures and call these through ctypes.
 *
 * Conventions (all entry points):
 *   - plain C, no C++ or torch types; returns 0 (TS_OK) or a negative TS_ERR_*;
 *   - every "dev" pointer is device memory owned by the caller and must stay
 *     alive until the work enqueued on `stream` has run;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - calls only enqueue work: no implicit synchronisation and no allocation;
 *     re-entrant from any thread.  State the library keeps: per thread, the
 *     HIP error of the last failed launch (ts_last_hip_error) and the event
 *     pair armed by ts_time_next_launch; per process, the address of the
 *     fixed scratch array of ts_kd_fwd_bwd_static, looked up once per GPU;
 *   - workspaces are caller-provided; sizes are stated per function;
 *   - a loss over zero rows (n_rows / n = 0) is accepted, its input and
 *     gradient pointers may then be null: loss = NaN, a mean over nothing, as
 *     the reference's kl_div 'batchmean', cross entropy and row means give;
 *   - "plan" functions are pure host code (no GPU needed): they turn tensor
 *     lists into the chunk tables the kernels walk.
 */
#ifndef TSPIPE_AMD_H
#define TSPIPE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ts_stream_t; /* hipStream_t */

enum ts_status {
  TS_OK = 0,
  TS_ERR_ARG = -1,      /* null pointer, negative size, unsupported dtype ... */
  TS_ERR_CAPACITY = -2, /* a plan does not fit the table the caller passed */
  TS_ERR_LAUNCH = -3,   /* hipLaunchKernel / hipFuncSetAttribute reported an error */
  TS_ERR_ALIGN = -4,    /* pointer not aligned to its element size */
  TS_ERR_RANGE = -5     /* size beyond what the kernel's grid/index type covers */
};

enum ts_dtype { TS_F32 = 0, TS_BF16 = 1, TS_F16 = 2 };

/* Library identification and error text (static strings). */
const char* ts_version(void);
const char* ts_error_string(int status);
/* Last HIP error code recorded by a failed launch in this thread (0 if none). */
int ts_last_hip_error(void);
/* Measurement aid, no counterpart in the reference.  Arms the calling thread:
 * the next kernel launched by ts_ema_multi, ts_ema_clone_multi or
 * ts_copy_segments from this thread records its own begin and end timestamps
 * into the two HIP events (hipEvent_t, created with timing enabled), as
 * hipExtLaunchKernel does; hipEventElapsedTime(start, stop) is then the
 * kernel's duration without the marker packets an event pair recorded around
 * the call would add.  Passing two nulls disarms. */
int ts_time_next_launch(void* start_event, void* stop_event);

/* ------------------------------------------------------------------------ */
/* Momentum-teacher EMA over a whole parameter list, one launch.         */
/*                                                                          */
/* Replaces the per-tensor loop                                              */
/*     detached = param_k.clone().detach()                                   */
/*     detached = detached * m + param_q.data * (1. - m)                     */
/* of benchmarks/byol/trainer.py:198-212 and benchmarks/moco-v3/main.py:     */
/* 133-144 (in-place twins: byol/trainer.py:43-49, moco/builder.py:57-61).   */
/* Arithmetic: out = fl32(fl32(t*m32) + fl32(s*c32)), no FMA contraction,    */
/* m32 = (float)m, c32 = (float)(1.0 - m) with the subtraction in double --  */
/* the rounding order of the eager fp32 ops, so results are bit-identical.   */
/* ------------------------------------------------------------------------ */

typedef struct ts_ema_chunk {
  const float* t; /* teacher (previous target) values of this chunk */
  const float* s; /* student (online) values */
  float* out;     /* new teacher values; may alias t for the in-place form */
  uint32_t n;     /* elements in the chunk (<= chunk_elems) */
  uint32_t flags; /* bit0: t, s and out are all 16-byte aligned */
} ts_ema_chunk;   /* 32 bytes */

/* Chunk size the planner picks for `total` elements when chunk_elems == 0. */
int64_t ts_ema_auto_chunk(int64_t total_elems);

/* Host: split n_tensors (t[i], s[i], out[i], numel[i]) into chunks.
 * chunk_elems: elements per chunk, a positive multiple of 1024, or 0 = the
 * value of ts_ema_auto_chunk(sum of numel).
 * table == NULL: only count.  Returns the chunk count (>= 0) or TS_ERR_*.
 * Tensors with numel 0 produce no chunk.  Pointers must be 4-byte aligned. */
int64_t ts_ema_plan(const void* const* t, const void* const* s, void* const* out,
                    const int64_t* numel, int64_t n_tensors, int64_t chunk_elems,
                    ts_ema_chunk* table, int64_t capacity);

/* Device: run the EMA over a table that lives in device memory.  chunk_elems
 * is the chunk size the table was planned with (the kernel cuts every chunk
 * into workgroup-sized pieces of 1024 elements). */
int ts_ema_multi(const ts_ema_chunk* table_dev, int64_t n_chunks, int64_t chunk_elems, float m32,
                 float c32, ts_stream_t stream);

/* The same two calls for parameter lists in another floating type (the
 * reference's per-tensor expression works on whatever dtype the parameters
 * have): dtype TS_F32, TS_BF16 or TS_F16, the same for t, s and out.  The
 * table's pointers are then element pointers of that type (for TS_F32 the
 * calls are ts_ema_plan / ts_ema_multi themselves).  Arithmetic as the eager
 * ops do it for a 2-byte type: each product and the sum are formed in fp32 and
 * rounded to the type, out = r(r(t*m32) + r(s*c32)).  Pointers must be aligned
 * to the element size; chunk_elems is a positive multiple of 2048 for the
 * 2-byte types (or 0 = automatic). */
int64_t ts_ema_plan_dtype(const void* const* t, const void* const* s, void* const* out,
                          const int64_t* numel, int64_t n_tensors, int64_t chunk_elems, int dtype,
                          ts_ema_chunk* table, int64_t capacity);
int ts_ema_multi_dtype(const ts_ema_chunk* table_dev, int64_t n_chunks, int64_t chunk_elems, float m32,
                       float c32, int dtype, ts_stream_t stream);

/* The same launch, also writing a clone of the student values: for every
 * chunk, s is copied to (char*)out + clone_offset_bytes.  Fuses the pipeline's
 * `online_new_param = [t.detach().clone() for t in online_prev_param]`
 * (tspipe/gpu_task.py:398) into the EMA that follows it (403-406), so the
 * optimizer-step tail moves 16 B per parameter instead of 8 + 12.  The caller
 * lays the clone buffer out exactly like the EMA output buffer (same offsets),
 * which is what makes one offset enough; clone_offset_bytes is a non-zero
 * multiple of 4 (of 16 for the vector path). */
int ts_ema_clone_multi(const ts_ema_chunk* table_dev, int64_t n_chunks, int64_t chunk_elems, float m32,
                       float c32, int64_t clone_offset_bytes, ts_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Multi-segment copy: micro-batch gather (torch.cat on dim 0,      */
/* tspipe/batch_ops.py:186-205, tspipe/utils.py:280), the owning form of     */
/* scatter (batch_ops.py:168-183), the student-parameter clone               */
/* (tspipe/gpu_task.py:398) and the teacher copy-in (gpu_task.py:706-724).   */
/* Byte-exact for any dtype.                                                 */
/* ------------------------------------------------------------------------ */

typedef struct ts_copy_chunk {
  const void* src;
  void* dst;
  uint64_t bytes;
  uint64_t flags; /* bit0: src and dst are both 16-byte aligned */
} ts_copy_chunk;  /* 32 bytes */

int64_t ts_copy_auto_chunk(int64_t total_bytes);

/* Host: split n_segments (src[i], dst[i], bytes[i]) into chunks of at most
 * chunk_bytes (positive multiple of 4096, or 0 = ts_copy_auto_chunk(sum)).  Same return rule as
 * ts_ema_plan.  Source and destination ranges must not overlap. */
int64_t ts_copy_plan(const void* const* src, void* const* dst, const int64_t* bytes,
                     int64_t n_segments, int64_t chunk_bytes, ts_copy_chunk* table,
                     int64_t capacity);

/* chunk_bytes: the chunk size the table was planned with. */
int ts_copy_segments(const ts_copy_chunk* table_dev, int64_t n_chunks, int64_t chunk_bytes,
                     ts_stream_t stream);

/* The same copy for up to 16 segments without a table: src, dst, bytes are
 * HOST arrays of n_segments entries (device pointers, byte counts; zero-length
 * segments are skipped) that travel in the kernel's arguments, so nothing is
 * planned or uploaded first.  For the small gathers of a pipeline -- the
 * torch.cat of a few micro-batch outputs of some kilobytes each,
 * tspipe/batch_ops.py:192,198 -- where the table's upload costs more than the
 * copy.  More than 16 segments: TS_ERR_RANGE (use the table). */
int ts_copy_few(const void* const* src, void* const* dst, const int64_t* bytes, int n_segments,
                ts_stream_t stream);

/* ------------------------------------------------------------------------ */
/* KD soft-target loss, forward and backward in one pass over rows.   */
/*                                                                          */
/* Replaces F.kl_div(F.log_softmax(s/T,1), F.softmax(t/T,1), 'batchmean')    */
/* * T * T (benchmarks/soft_target/kd_losses/st.py:18-23) and the masked     */
/* wide-vocabulary form of benchmarks/distilbert/distiller.py:719-740        */
/* (masked_select of rows, KLDivLoss('batchmean'), * temperature**2).        */
/*                                                                          */
/*   B       = number of rows with row_mask != 0 (all n_rows if mask NULL)   */
/*   loss    = loss_scale / B * sum_rows KL(softmax(t/T) || softmax(s/T))    */
/*   grad_ij = loss_scale * inv_T / B * (q_ij - p_ij) for selected rows,     */
/*             0 for the others (dense, like masked_select's backward)       */
/* with loss_scale = T*T*weight chosen by the caller.  B == 0 gives          */
/* loss = NaN and grad = 0, as the reference's 0/0 does.                     */
/*                                                                          */
/* s, t, grad: [n_rows, V] row-major with leading dimensions ld_* in         */
/* elements; dtype TS_F32 / TS_BF16 / TS_F16 (same for all three);           */
/* accumulation is fp32.  grad may be NULL (loss only).                      */
/* workspace: ts_kd_workspace_bytes(n_rows, V, dtype) bytes, 32-byte aligned,  */
/* contents irrelevant on entry.  loss_out: one float.                       */
/* ------------------------------------------------------------------------ */

size_t ts_kd_workspace_bytes(int64_t n_rows, int64_t V, int dtype);

int ts_kd_fwd_bwd(const void* s, const void* t, const uint8_t* row_mask, int64_t n_rows,
                  int64_t V, int64_t ld_s, int64_t ld_t, float inv_T, float loss_scale,
                  void* workspace, float* loss_out, void* grad, int64_t ld_g, int dtype,
                  ts_stream_t stream);

/* ts_kd_fwd_bwd for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc): no
 * counterpart in the reference.  Same arguments without the workspace, same
 * kernels and results; the workspace is a fixed array inside the library
 * (ts_kd_static_scratch_bytes() bytes, one copy per GPU, held until the
 * process ends).  Shapes whose ts_kd_workspace_bytes() exceeds that size are
 * refused with TS_ERR_RANGE.  The call allocates nothing.  Every call on a GPU
 * uses that GPU's one array: calls that may overlap on the same GPU (two
 * streams, two threads) race and must be serialised by the caller. */
size_t ts_kd_static_scratch_bytes(void);

int ts_kd_fwd_bwd_static(const void* s, const void* t, const uint8_t* row_mask, int64_t n_rows,
                         int64_t V, int64_t ld_s, int64_t ld_t, float inv_T, float loss_scale,
                         float* loss_out, void* grad, int64_t ld_g, int dtype, ts_stream_t stream);

/* The same pass with the hard-label cross entropy added, the combination the
 * reference's distillation plug-ins compute on the student logits:
 *   benchmarks/soft_target/train_kd.py:439-453
 *       CrossEntropyLoss()(model_out, label) + SoftTarget(T)(model_out, ema_out) * lambda_kd
 *   benchmarks/distilbert/distiller.py:719-744
 *       alpha_ce * KLDiv(masked rows) * T^2 + alpha_mlm * CrossEntropyLoss(ignore_index=-100)(all rows, lm_labels)
 *
 *   loss = kd_scale / B_kd * sum_{rows with row_mask} KL(...)
 *        + ce_weight / B_ce * sum_{rows with a valid label} (logsumexp(s_row) - s_row[label])
 * B_kd as in ts_kd_fwd_bwd; B_ce = rows whose label differs from ignore_index
 * (labels outside [0, V) are treated as ignored).  The two row sets are
 * independent; rows in neither get a zero gradient.  labels: int64 per row, or
 * NULL for no CE term (then identical to ts_kd_fwd_bwd with loss_scale =
 * kd_scale).  Same workspace as ts_kd_fwd_bwd. */
int ts_kdce_fwd_bwd(const void* s, const void* t, const uint8_t* row_mask, const int64_t* labels,
                    int64_t ignore_index, int64_t n_rows, int64_t V, int64_t ld_s, int64_t ld_t,
                    float inv_T, float kd_scale, float ce_weight, void* workspace, float* loss_out,
                    void* grad, int64_t ld_g, int dtype, ts_stream_t stream);

/* The same loss on logits that were never concatenated: the student and teacher
 * outputs of up to 8 micro-batches stay where the pipeline produced them
 * (tspipe/gpu_task.py:147,170-171,188-191 concatenates them with torch.cat
 * before calling loss_fn; this entry point makes both copies unnecessary) and
 * the gradient is written straight into one buffer per piece.
 *   s_pieces, t_pieces, grad_pieces: host arrays of n_pieces device pointers,
 *     piece p being a contiguous [piece_rows[p], V] matrix; grad_pieces may be
 *     NULL (or hold NULLs) for loss only;
 *   row_mask, labels: device arrays over the rows of all pieces in order
 *     (sum of piece_rows entries), as for ts_kdce_fwd_bwd; either may be NULL.
 * workspace: ts_kd_workspace_bytes(sum of piece_rows, V, dtype).  More than 8
 * pieces: TS_ERR_RANGE (gather first, or call once per group of pieces). */
int ts_kdce_pieces_fwd_bwd(const void* const* s_pieces, const void* const* t_pieces,
                           void* const* grad_pieces, const int64_t* piece_rows, int n_pieces,
                           const uint8_t* row_mask, const int64_t* labels, int64_t ignore_index,
                           int64_t V, float inv_T, float kd_scale, float ce_weight,
                           void* workspace, float* loss_out, int dtype, ts_stream_t stream);

/* grad *= *g for the rows the loss touched; returns at once on the device
 * when *g == 1 (the only value TSPipe's torch.autograd.backward(loss) feeds,
 * tspipe/gpu_task.py:207-212).  g_dev: one float in device memory. */
int ts_scale_rows(void* grad, int64_t n_rows, int64_t V, int64_t ld_g, const float* g_dev,
                  int dtype, ts_stream_t stream);

/* ------------------------------------------------------------------------ */
/* BYOL normalised-MSE loss, forward and backward.                       */
/*                                                                          */
/* Replaces regression_loss (benchmarks/byol/trainer.py:51-55) and           */
/* contrastive_loss (trainer.py:192-196):                                    */
/*   rl(x,y)_i = 2 - 2 * <x_i/max(|x_i|,1e-12), y_i/max(|y_i|,1e-12)>        */
/*   loss = mean_i( rl(x1,y1)_i + rl(x2,y2)_i )      (x2,y2 may be NULL)     */
/*   gx   = d loss / d x  (teacher side y gets no gradient)                  */
/* x*, y*, gx*: [n, c] contiguous, same dtype.  workspace: 2*n floats.       */
/* ------------------------------------------------------------------------ */

int ts_byol_fwd_bwd(const void* x1, const void* y1, const void* x2, const void* y2, int64_t n,
                    int64_t c, float* workspace, float* loss_out, void* gx1, void* gx2,
                    int dtype, ts_stream_t stream);

/* The same loss on projections that were never concatenated: x, y and gx of
 * each pair come as up to 8 row blocks (the micro-batch outputs that
 * tspipe/gpu_task.py:188-191 concatenates with torch.cat before calling
 * loss_fn); the gradient goes straight into one buffer per piece.  Host arrays
 * of n_pieces device pointers, piece p being a contiguous [piece_rows[p], c]
 * matrix; the second pair's arrays may be NULL; the gx arrays may be NULL (or
 * hold NULLs) for loss only.  workspace: 2 * (sum of piece_rows) floats.
 * More than 8 pieces: TS_ERR_RANGE. */
int ts_byol_pieces_fwd_bwd(const void* const* x1_pieces, const void* const* y1_pieces,
                           void* const* gx1_pieces, const void* const* x2_pieces,
                           const void* const* y2_pieces, void* const* gx2_pieces,
                           const int64_t* piece_rows, int n_pieces, int64_t c, float* workspace,
                           float* loss_out, int dtype, ts_stream_t stream);

/* Squared error between student and teacher logits, forward and backward:
 *   Logits.forward (benchmarks/soft_target/kd_losses/logits.py:17-20), F.mse_loss
 *     with its mean over all elements: per_element = 1, row_mask = NULL;
 *   the alpha_mse term of DistilBERT's loss (benchmarks/distilbert/distiller.py:751-755),
 *     MSELoss(reduction="sum") over the rows the mask keeps, divided by their
 *     number: per_element = 0.
 *   loss = weight * sum_{rows with row_mask != 0} sum_v (s - t)^2 / denom,
 *   denom = selected rows (x V if per_element);  grad = d loss / d s, zero on
 *   the other rows.  accumulate != 0 adds loss and gradient to what loss_out
 *   and grad already hold (the term joins a KD gradient in place) and leaves
 *   unselected rows untouched.
 * s, t, grad: [n_rows, V] with leading dimensions; grad may be NULL.
 * workspace: ts_mse_workspace_bytes(n_rows, V) bytes, 16-byte aligned. */
size_t ts_mse_workspace_bytes(int64_t n_rows, int64_t V);

int ts_mse_fwd_bwd(const void* s, const void* t, const uint8_t* row_mask, int64_t n_rows, int64_t V,
                   int64_t ld_s, int64_t ld_t, float weight, int per_element, int accumulate,
                   void* workspace, float* loss_out, void* grad, int64_t ld_g, int dtype,
                   ts_stream_t stream);

/* The same term on logits that were never concatenated (the micro-batch
 * outputs that tspipe/gpu_task.py:188-191 concatenates before calling loss_fn;
 * the term itself is benchmarks/distilbert/distiller.py:751-755): host arrays
 * of n_pieces device pointers, piece p being a contiguous [piece_rows[p], V]
 * matrix; row_mask covers all rows in order; grad_pieces may be NULL (or hold
 * NULLs) for loss only.  workspace: ts_mse_workspace_bytes(sum of piece_rows, V).
 * More than 8 pieces: TS_ERR_RANGE. */
int ts_mse_pieces_fwd_bwd(const void* const* s_pieces, const void* const* t_pieces,
                          void* const* grad_pieces, const int64_t* piece_rows, int n_pieces,
                          const uint8_t* row_mask, int64_t V, float weight, int per_element,
                          int accumulate, void* workspace, float* loss_out, int dtype,
                          ts_stream_t stream);

/* Cosine embedding loss with target +1, forward and backward: the hidden-state
 * term of DistilBERT's loss (benchmarks/distilbert/distiller.py:756-770,
 * nn.CosineEmbeddingLoss(reduction="mean") on the rows the attention mask keeps):
 *   cos_i = <x_i, y_i> / sqrt((|x_i|^2 + 1e-12)(|y_i|^2 + 1e-12))
 *   loss  = weight * mean over rows with row_mask != 0 of (1 - cos_i)
 *   gx    = d loss / d x, zero for the other rows (y is the detached teacher)
 * x, y, gx: [n, c] contiguous; row_mask may be NULL (all rows); gx may be NULL.
 * workspace: ts_cosine_workspace_bytes(n) bytes, 16-byte aligned. */
size_t ts_cosine_workspace_bytes(int64_t n);

int ts_cosine_fwd_bwd(const void* x, const void* y, const uint8_t* row_mask, int64_t n, int64_t c,
                      float weight, void* workspace, float* loss_out, void* gx, int dtype,
                      ts_stream_t stream);

/* The same loss on hidden states that were never concatenated
 * (tspipe/gpu_task.py:188-191; the term is distiller.py:756-770): host arrays
 * of n_pieces device pointers, piece p being a contiguous [piece_rows[p], c]
 * matrix; row_mask covers all rows in order; gx_pieces may be NULL (or hold
 * NULLs) for loss only.  workspace: ts_cosine_workspace_bytes(sum of
 * piece_rows).  More than 8 pieces: TS_ERR_RANGE. */
int ts_cosine_pieces_fwd_bwd(const void* const* x_pieces, const void* const* y_pieces,
                             void* const* gx_pieces, const int64_t* piece_rows, int n_pieces,
                             const uint8_t* row_mask, int64_t c, float weight, void* workspace,
                             float* loss_out, int dtype, ts_stream_t stream);

/* ------------------------------------------------------------------------ */
/* MoCo-v3 InfoNCE loss, forward and backward, logits never stored.      */
/*                                                                          */
/* Replaces contrastive_loss.loss (benchmarks/moco-v3/main.py:147-162;       */
/* single-device twin moco/builder.py:63-71):                                */
/*   qh = q/max(|q|,1e-12), kh likewise; logits = qh kh^T / tau;             */
/*   loss = CrossEntropy(logits, arange(N)) * 2 tau   (mean over rows)       */
/*   dq   = d loss / d q  (k is the detached teacher output)                 */
/* Up to two (q,k) pairs are summed into one loss (main.py:162); q2,k2,dq2   */
/* may be NULL.  q*, k*: [n, c] contiguous, 1 <= c <= 512 (--moco-dim,        */
/* main.py:98), any tau > 0 (--moco-t, main.py:107); dq comes back in the     */
/* input type.  Two implementations, chosen per call:                        */
/*   bf16 MFMA: TS_BF16 / TS_F16 inputs (fp16 rounded to bf16 for the         */
/*     contraction) with c = 64, 128 or 256, tau >= 0.03 and rows on 16-byte  */
/*     boundaries;                                                            */
/*   fp32 MFMA: everything else -- TS_F32 inputs (the reference's TSPipe run  */
/*     is fp32, main.py:151-160), other widths, smaller temperatures; every   */
/*     product and sum in fp32, running row maximum.                          */
/* workspace: ts_infonce_workspace_bytes(n, c, n_pairs) bytes, 256-aligned    */
/* (covers either implementation).                                           */
/* ------------------------------------------------------------------------ */

size_t ts_infonce_workspace_bytes(int64_t n, int64_t c, int n_pairs);

/* No counterpart in the reference: a scheduling knob for callers that run the
 * loss beside other GPU work, as TSPipe's pipeline does (the loss of one
 * micro-batch beside the momentum update and the next forward,
 * tspipe/gpu_task.py:385-410).  The main kernels cut the keys into as many
 * splits as it takes to put about `workgroups` workgroups on the chip; every
 * split writes partial sums that the last launch adds up.  The default, 256
 * (one per CU), makes a call that has the GPU to itself fastest.  A smaller
 * number means fewer, longer workgroups: fewer partial sums through HBM and
 * CUs left to whatever runs on the other streams, at the price of a longer
 * loss kernel.  Results agree to rounding (the partial sums are added in split
 * order either way).  Process-wide; values outside 1..256 restore the default.
 * Returns the previous value.  ts_infonce_workspace_bytes does not depend on
 * it. */
int ts_infonce_set_workgroup_target(int workgroups);

/* No counterpart in the reference: an accuracy switch.  With on != 0 every
 * call takes the fp32-MFMA implementation, also for TS_BF16 / TS_F16 inputs of
 * 64, 128 or 256 features: products and sums in fp32, nothing rounded to bf16
 * on the way, at about seven times the time of the bf16-MFMA implementation
 * (4096 x 256: 0.23 ms against 0.035 ms).  For callers whose embeddings are
 * nearly aligned with their keys (a trained model), where the bf16 rounding of
 * the negatives' weights is what is left of the gradient's error.  Process-wide;
 * returns the previous setting (0 or 1).  The workspace size does not depend
 * on it. */
int ts_infonce_set_fp32_arithmetic(int on);

int ts_infonce_fwd_bwd(const void* q1, const void* k1, const void* q2, const void* k2, int64_t n,
                       int64_t c, float tau, void* workspace, float* loss_out, void* dq1,
                       void* dq2, int dtype, ts_stream_t stream);

/* The same loss on embeddings that were never concatenated: q, k and dq of
 * each pair come as up to 8 row blocks (the micro-batch outputs that
 * tspipe/gpu_task.py:170-171,188-191 concatenates with torch.cat before calling
 * loss_fn; the gradient goes straight into one buffer per piece).
 *   q1_pieces, k1_pieces, dq1_pieces (and the second pair's, or NULLs): host
 *     arrays of n_pieces device pointers, piece p being a contiguous
 *     [piece_rows[p], c] matrix (16-byte aligned for the bf16 implementation,
 *     element-aligned otherwise); the dq arrays may be NULL
 *     (or hold NULLs) for loss only.  Both pairs share piece_rows.
 * workspace: ts_infonce_workspace_bytes(sum of piece_rows, c, n_pairs).
 * More than 8 pieces: TS_ERR_RANGE. */
int ts_infonce_pieces_fwd_bwd(const void* const* q1_pieces, const void* const* k1_pieces,
                              void* const* dq1_pieces, const void* const* q2_pieces,
                              const void* const* k2_pieces, void* const* dq2_pieces,
                              const int64_t* piece_rows, int n_pieces, int64_t c, float tau,
                              void* workspace, float* loss_out, int dtype, ts_stream_t stream);

/* ------------------------------------------------------------------------ */
/* DeferredBatchNorm (tspipe/batchnorm.py).                           */
/* x, y, dy, dx: fp32 [N, C, HW] contiguous (NCHW with HW = prod of the      */
/* trailing dims).  Two families of kernels behind every call: planes of     */
/* more than 256 elements are dealt a wavefront each; smaller ones (the late  */
/* stages of a ResNet, [N, C, 1, 1]) are walked as flat ranges of a sample    */
/* when C*HW is a multiple of 4 and the tensors sit on 16-byte boundaries.    */
/* ------------------------------------------------------------------------ */

/* _track (batchnorm.py:45-59) fused with the statistics F.batch_norm(
 * training=True) needs (batchnorm.py:111-120): one read of x gives the
 * micro-batch's per-channel sum and sum of squares, which are
 *   - added into the mini-batch accumulators `sum`, `sum_squares` (fp32 +=),
 *     unless those are NULL;
 *   - turned into ub_mean = S/cnt and ub_invstd = 1/sqrt(max(Q/cnt - mean^2,0)
 *     + eps), cnt = N*HW, unless those are NULL.
 * One launch: the last workgroup of a channel to finish does the channel's
 * bookkeeping (small planes: two short launches).  ws: ts_bn_stats_workspace_bytes(C) bytes (3*C floats: two
 * sums and a ticket counter per channel) that are ZERO on entry; the call
 * leaves them zero again.  Calls that share a ws must not overlap on the
 * device (the last workgroup of a channel reads and clears what the others
 * added): keep them on one stream, or order the streams with events.  A
 * buffer of the 2*C floats that an earlier version of this call asked for is
 * too small.  x is fetched with non-temporal loads (it is not read again by
 * this call): a caller that goes on to normalise the same x should use
 * ts_bn_forward_train, whose statistics half leaves x to its second half in
 * the caches. */
size_t ts_bn_stats_workspace_bytes(int64_t C);

int ts_bn_stats(const float* x, int64_t N, int64_t C, int64_t HW, float* ws, float* sum,
                float* sum_squares, float* ub_mean, float* ub_invstd, float eps,
                ts_stream_t stream);

/* _commit (batchnorm.py:61-85): num_batches_tracked += 1;
 * f = momentum, or 1/num_batches_tracked when momentum < 0 (the reference's
 * momentum=None); mean = sum/counter; var = sum_squares/counter - mean^2;
 * running = running*(1-f) + stat*f in the reference's fp32 rounding order;
 * then sum = sum_squares = 0. */
int ts_bn_commit(float* sum, float* sum_squares, float* running_mean, float* running_var,
                 int64_t* num_batches_tracked, int64_t C, double counter, double momentum,
                 ts_stream_t stream);

/* y = (x - mean[c]) * invstd[c] * gamma[c] + beta[c]; gamma/beta may be NULL
 * (affine=False).  With is_var != 0 the fourth argument holds variances and
 * invstd = 1/sqrt(var + eps) is formed on the fly (eval mode with running
 * statistics, batchnorm.py:88-99). */
int ts_bn_apply(const float* x, float* y, const float* mean, const float* invstd_or_var,
                const float* gamma, const float* beta, int64_t N, int64_t C, int64_t HW,
                int is_var, float eps, ts_stream_t stream);

/* Training forward of one micro-batch in two launches instead of three:
 * ts_bn_stats + ts_bn_apply(training) with the bookkeeping of the statistics
 * folded into the normalising kernel (tspipe/batchnorm.py:45-59 and 111-120
 * together).  Same results as the two calls, bit for bit.
 *   ws: 4*C floats, zero before the first call, owned by the layer: two
 *       halves used alternately.  parity (0/1) selects the half this call
 *       reduces into; it must alternate from call to call on the same ws
 *       (the call clears the half the previous call used).
 *   sum, sum_squares, ub_mean, ub_invstd: as for ts_bn_stats (any may be NULL). */
int ts_bn_forward_train(const float* x, float* y, const float* gamma, const float* beta, int64_t N,
                        int64_t C, int64_t HW, float* sum, float* sum_squares, float* ub_mean,
                        float* ub_invstd, float* ws, int parity, float eps, ts_stream_t stream);

/* Backward of the normalisation (what autograd derives for F.batch_norm):
 * dgamma = sum dy*xhat, dbeta = sum dy, and
 *   training != 0 (batch statistics, batchnorm.py:111-120):
 *     dx = gamma*invstd*(dy - dbeta/cnt - xhat*dgamma/cnt)
 *   training == 0 (fixed running statistics, batchnorm.py:88-99):
 *     dx = gamma*invstd*dy
 * Two launches: the reduction, then dx, whose workgroups read the two sums
 * themselves.  ws, parity: as for ts_bn_forward_train (4*C floats, zero before
 * the first use, two halves used alternately; a layer's forward and backward
 * calls may share one ws and one alternating parity).  dgamma/dbeta: [C]
 * outputs (required); gamma may be NULL (treated as 1). */
int ts_bn_backward(const float* x, const float* dy, const float* ub_mean, const float* ub_invstd,
                   const float* gamma, float* dx, float* dgamma, float* dbeta, float* ws, int parity,
                   int64_t N, int64_t C, int64_t HW, int training, ts_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TSPIPE_AMD_H */
