/*
 * picotron_amd -- C ABI of the MI355X (gfx950) hot-path library  libpicotron_amd.so
 *
 * picotron has no FFI of its own: the path it accelerates is a set of Python functions
 * (picotron/context_parallel/context_parallel.py, picotron/model.py) that call torch /
 * flash-attn ops.  Each entry point below replaces the arithmetic of one of those call
 * sites; the citation after "replaces:" is the reference file:line.
 *
 * Conventions
 *  - plain pointers to DEVICE memory + sizes; no torch types.  The library never allocates,
 *    frees or synchronises: every call only enqueues kernels on `stream` (a hipStream_t,
 *    passed as void*; NULL = the default stream).  Safe to call from any host thread.
 *  - every function returns PICO_OK (0) or a negative pico_status; the text of the last
 *    failure on the calling thread is available from pico_last_error().
 *  - tensors are addressed as [B, H, S, D] with explicit element strides for (b, h, s) and a
 *    unit stride on D, so both a contiguous [B,H,S,D] buffer and a transposed view of a
 *    [B,S,H,D] buffer (what picotron's Attention produces, model.py:128-130) are accepted.
 *  - dtype codes: PICO_BF16 / PICO_F32.  Attention operands are bf16 only.
 */
#ifndef PICOTRON_AMD_H
#define PICOTRON_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum pico_status {
  PICO_OK = 0,
  PICO_ERR_NULL = -1,      /* a required pointer is NULL */
  PICO_ERR_DTYPE = -2,     /* unsupported dtype code */
  PICO_ERR_SHAPE = -3,     /* unsupported size (head_dim, hidden, negative dims, GQA ratio) */
  PICO_ERR_ALIGN = -4,     /* pointer or stride not aligned as the kernel needs */
  PICO_ERR_STRIDE = -5,    /* stride combination not supported */
  PICO_ERR_WORKSPACE = -6, /* workspace too small */
  PICO_ERR_LAUNCH = -7     /* hipLaunchKernel reported an error */
} pico_status;

typedef enum pico_dtype { PICO_BF16 = 0, PICO_F32 = 1 } pico_dtype;

/* Library version string, e.g. "picotron_amd 0.1 gfx950". */
const char* pico_version(void);
/* Message of the last failing call made by this thread ("" if none). */
const char* pico_last_error(void);

/* ------------------------------------------------------------------ RMSNorm
 * replaces: LlamaRMSNorm.forward  model.py:81-86  (cast_then_scale = 1: the normalised value is
 *           rounded to the io dtype, then multiplied by the weight in that dtype)
 *           TritonRMSNorm.forward model.py:51-65 -> flash-attn layer_norm_fn(is_rms_norm=True)
 *           (cast_then_scale = 0: fp32 maths, one rounding).
 * x, y: [rows, hidden] contiguous, dtype `dtype`; weight: [hidden] same dtype.
 * rstd: optional [rows] fp32 output (1/sqrt(mean x^2 + eps)), saved for the backward.
 * residual_in / residual_out: optional fused pre-norm residual add (TritonRMSNorm's
 *   residual= / prenorm= arguments): h = x + residual_in is normalised and, if residual_out is
 *   given, written there in the io dtype.  Pass NULL for both to get the plain norm.
 * hidden must be a multiple of 8 (bf16) / 4 (fp32) and <= 16384.
 */
int pico_rmsnorm_fwd(const void* x, const void* weight, void* y, float* rstd,
                     const void* residual_in, void* residual_out,
                     int64_t rows, int64_t hidden, float eps, int cast_then_scale,
                     int dtype, void* stream);

/* Bytes of fp32 workspace pico_rmsnorm_bwd needs for the per-block partial sums of dweight. */
int64_t pico_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t hidden);

/* replaces: autograd of model.py:81-86 / the Triton backward of layer_norm_fn.
 * dx = rstd * (g - xhat * mean(g * xhat)),  g = dy * w,  xhat = x * rstd;  dweight = sum_rows dy * xhat.
 * x is the tensor that was normalised (after the residual add, if any).
 * dresidual: optional [rows, hidden] `dtype`, added to dx -- the gradient that reached the residual stream directly
 *   when the forward fused the residual add (the dresidual input of layer_norm_fn's backward); dx may alias it.
 * dx: [rows, hidden] `dtype` (may alias dy); dweight: [hidden] of dweight_dtype (PICO_F32 or PICO_BF16; summed in fp32
 *   and rounded once, the rows' contributions always in the same order: no atomics, equal inputs give equal bits);
 *   workspace: device scratch of at least pico_rmsnorm_bwd_workspace_bytes() bytes (contents undefined on entry and
 *   exit).
 */
int pico_rmsnorm_bwd(const void* dy, const void* x, const void* weight, const float* rstd, const void* dresidual,
                     void* dx, void* dweight, int dweight_dtype, void* workspace, int64_t workspace_bytes,
                     int64_t rows, int64_t hidden, int dtype, void* stream);

/* pico_rmsnorm_bwd without the workspace argument: the one entry point that allocates nothing and needs nothing
 * allocated for it.  It has no counterpart in the reference; it is for callers that cannot call hipMalloc or hand over
 * scratch memory -- code under HIP graph capture, tight serving loops, harnesses that forbid allocation.  The
 * per-block partial sums of dweight go to a static device array inside the library (4 MiB per GPU, held until the
 * process ends) instead of the caller's workspace; arguments, kernels and results are otherwise those of
 * pico_rmsnorm_bwd, bit for bit.  The device the pointers live on must be the current device.
 * Limit: the launch's partial sums must fit the array -- pico_rmsnorm_bwd_static_max_bytes(); every hidden <= 16384
 * the kernels accept does, whatever `rows` is -- otherwise PICO_ERR_WORKSPACE is returned and nothing is launched.
 * All calls on one GPU share that array: calls that overlap in time on one GPU (two streams, two host threads)
 * race on it and must be serialised by the caller.  Nothing in it needs clearing between calls: a launch writes
 * every partial sum it later reads.
 */
int64_t pico_rmsnorm_bwd_static_max_bytes(void);
int pico_rmsnorm_bwd_static(const void* dy, const void* x, const void* weight, const float* rstd,
                            const void* dresidual, void* dx, void* dweight, int dweight_dtype,
                            int64_t rows, int64_t hidden, int dtype, void* stream);

/* ------------------------------------------------------------------ RoPE
 * replaces: apply_rotary_pos_emb  model.py:12-19  and the flash-attn rotary call model.py:136-137
 *           (non-interleaved: element i pairs with i + D/2), with the row selection of
 *           update_rope_for_context_parallel  context_parallel.py:189-195 folded in as pos_offset.
 * y[b,h,s,:D/2] = x1*cos - x2*sin ; y[b,h,s,D/2:] = x2*cos + x1*sin,  cos/sin row = pos_offset + s.
 * cos, sin: [>= pos_offset + S, table_ld] tables of dtype table_dtype; only the first D/2 columns
 * are read (get_cos_sin duplicates the halves, model.py:31).  x and y may alias (in place).
 * inverse = 1 applies the rotation by -theta, which is the backward (adjoint) of the forward.
 * D must be a multiple of 16 and <= 256; strides in elements, D contiguous.
 */
int pico_rope(const void* x, void* y, const void* cos, const void* sin,
              int64_t B, int64_t H, int64_t S, int64_t D,
              int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_s,
              int64_t y_stride_b, int64_t y_stride_h, int64_t y_stride_s,
              int64_t table_ld, int64_t pos_offset, int inverse,
              int table_dtype, int dtype, void* stream);

/* ------------------------------------------------------------------ SwiGLU activation
 * replaces: F.silu(gate) * up  model.py:186  and its autograd.
 * gate, up, y (and dy, dgate, dup): [rows, cols] with row pitches *_ld in elements; cols % 8 == 0.
 */
int pico_swiglu_fwd(const void* gate, const void* up, void* y,
                    int64_t rows, int64_t cols, int64_t gate_ld, int64_t up_ld, int64_t y_ld,
                    int dtype, void* stream);
int pico_swiglu_bwd(const void* dy, const void* gate, const void* up, void* dgate, void* dup,
                    int64_t rows, int64_t cols, int64_t dy_ld, int64_t gate_ld, int64_t up_ld,
                    int64_t dgate_ld, int64_t dup_ld, int dtype, void* stream);

/* ------------------------------------------------------------------ online-softmax merge
 * replaces: update_out_and_lse  context_parallel.py:157-187 (the _update branch, :170-171):
 *   out <- out - sigmoid(block_lse - lse) * (out - block_out);  lse <- lse - logsigmoid(lse - block_lse)
 * out: [rows, D] fp32 in/out; lse: [rows] fp32 in/out; block_out: [rows, D] of block_dtype;
 * block_lse: [rows] fp32.  rows = B*H*Sq.
 */
int pico_lse_merge(float* out, float* lse, const void* block_out, const float* block_lse,
                   int64_t rows, int64_t D, int block_dtype, void* stream);

/* ------------------------------------------------------------------ attention
 * One descriptor serves forward and backward.  q, k, v, dout are bf16.
 *   query i of the launch sits at absolute position q_offset + i, key j at position j;
 *   with causal != 0 key j is visible iff j <= q_offset + i.
 * q_offset = 0 and Sq == Sk is the masked diagonal block of the reference (context_parallel.py:116-119);
 * causal = 0 is a dense off-diagonal block; q_offset = r*Sc with Sk = (r+1)*Sc runs ALL ring steps
 * of cp rank r in one launch (the K/V chunks 0..r laid out consecutively along S).
 * Hq % Hkv == 0: query head h reads kv head h / (Hq/Hkv), i.e. the effect of the reference's
 * repeat_interleave (model.py:142-143) without the copy; pass Hkv == Hq for pre-expanded K/V.
 */
typedef struct pico_attn_desc {
  int32_t B, Hq, Hkv, Sq, Sk, D;   /* D in {64, 128} */
  int32_t causal;
  int32_t q_offset;
  float sm_scale;
  int32_t reserved;
  int64_t q_stride[3];             /* elements, order (b, h, s); D stride is 1 */
  int64_t k_stride[3];
  int64_t v_stride[3];
  int64_t o_stride[3];             /* out, and dout in the backward */
} pico_attn_desc;

/* replaces: ring_attention_forward  context_parallel.py:112-128  (merge = 0), and
 *           ring_attention_forward + update_out_and_lse  context_parallel.py:37-40 (merge = 1).
 * out:  [B,Hq,Sq,D] addressed by o_stride; dtype out_dtype (PICO_BF16 or PICO_F32).
 * lse:  [B,Hq,Sq] contiguous fp32.
 * merge = 1: (out, lse) hold the running fp32 result of earlier blocks on entry (out_dtype must be
 * PICO_F32) and the merged result on exit -- the online softmax simply continues from that state.
 * Rows that see no key get out = 0 and lse = -inf.
 */
int pico_attn_fwd(const pico_attn_desc* desc, const void* q, const void* k, const void* v,
                  void* out, float* lse, int out_dtype, int merge, void* stream);

/* RoPE tables for the attention entry points that rotate inside the kernel: cos / sin [rows, >= D/2 columns]
 * (get_cos_sin's tables, model.py:21-31: only the first D/2 columns are read), `pitch` elements between rows,
 * dtype PICO_BF16 or PICO_F32, row index = absolute position.
 */
typedef struct pico_rope_tables {
  const void* cos;
  const void* sin;
  int64_t pitch;
  int32_t dtype;
  int32_t rows;
} pico_rope_tables;

/* replaces: apply_rotary_pos_emb on q (model.py:131 / :136) followed by the attention forward (model.py:154-157):
 * q arrives UN-rotated and every query is rotated once, in the prologue of the workgroup that owns it
 * (position = q_pos_offset + row; fp32 arithmetic, one rounding, as pico_rope); k_rot must already be rotated
 * (pico_rope on k: a key tile is read by many workgroups, rotating it there would repeat the work).  If q_rot is
 * given the rotated q is written there (bf16, its own b/h/s strides with rows that do not overlap, unit D stride)
 * for pico_attn_bwd_rope.  merge as in pico_attn_fwd: with merge = 1 the call is one step of a ring whose queries
 * sit at positions q_pos_offset .. (update_rope_for_context_parallel, context_parallel.py:189-195, as an offset).
 * Everything else as pico_attn_fwd.
 */
int pico_attn_fwd_rope(const pico_attn_desc* desc, const void* q, const void* k_rot, const void* v, void* out,
                       float* lse, int out_dtype, int merge, const pico_rope_tables* rope, int q_pos_offset, void* q_rot,
                       const int64_t* q_rot_stride, void* stream);

/* replaces: D = sum(dO * O, dim=-1)  context_parallel.py:145.
 * delta: [B,Hq,Sq] fp32.  out is addressed by o_stride like dout and has dtype out_dtype.
 * If dq_acc is not NULL that [B,Hq,Sq,D] contiguous fp32 buffer is zeroed in the same pass (optional).
 */
int pico_attn_bwd_preprocess(const pico_attn_desc* desc, const void* dout, const void* out, int out_dtype,
                             float* delta, float* dq_acc, void* stream);

/* replaces: ring_attention_backward  context_parallel.py:130-155 and the fp32 accumulation of
 *           RingAttentionFunc.backward  context_parallel.py:85-93.
 * Two kernels are enqueued: dK/dV (one workgroup per 128 keys) and dQ (one workgroup per query tile);
 * neither uses atomics, so results are deterministic.
 * lse, delta: [B,Hq,Sq] fp32 (lse is the FINAL merged lse, as in the reference).
 * dq:     [B,Hq,Sq,D] addressed by dq_stride (element strides for b, h, s, multiples of 4; NULL = contiguous);
 *         dq_dtype PICO_F32 with dq_accumulate = 1 adds into the buffer (the running sum over ring steps),
 *         dq_accumulate = 0 overwrites; PICO_BF16 overwrites.
 * dk, dv: [B,Hkv,Sk,D] addressed by dkv_stride (multiples of 8; NULL = contiguous); same dtype / accumulate rules (the
 *         travelling fp32 accumulators of the ring).  With Hq > Hkv the group's query heads are reduced
 *         inside the kernel.
 * A gradient that is not wanted is passed as NULL (dq, or dk and dv together) and its kernel is skipped.
 */
int pico_attn_bwd(const pico_attn_desc* desc, const void* q, const void* k, const void* v,
                  const void* dout, const float* lse, const float* delta,
                  void* dq, const int64_t* dq_stride, int dq_dtype, int dq_accumulate,
                  void* dk, void* dv, const int64_t* dkv_stride, int dkv_dtype, int dkv_accumulate,
                  void* stream);

/* replaces: ring_attention_backward  context_parallel.py:130-155 as ONE call, delta = sum_d dO * O (:145) included.
 * Same arguments as pico_attn_bwd plus the forward output `out` (addressed by o_stride like dout, dtype out_dtype);
 * `delta` is an OUTPUT here: [B,Hq,Sq] fp32, written with the row sums.  With a bf16 `out` and a wanted dq the dQ
 * kernel computes delta in its prologue and runs before the dK/dV kernel (one launch and one pass over dO and O
 * less than pico_attn_bwd_preprocess + pico_attn_bwd); otherwise the pre-pass is enqueued internally.
 */
int pico_attn_bwd_fused(const pico_attn_desc* desc, const void* q, const void* k, const void* v,
                        const void* dout, const void* out, int out_dtype, const float* lse, float* delta,
                        void* dq, const int64_t* dq_stride, int dq_dtype, int dq_accumulate,
                        void* dk, void* dv, const int64_t* dkv_stride, int dkv_dtype, int dkv_accumulate,
                        void* stream);

/* replaces: the backward of "rotate q and k, then attend" (autograd of model.py:131-137 + :154-157):
 * pico_attn_bwd_fused on the ROTATED q and k (q_rot as written by pico_attn_fwd_rope, k_rot from pico_rope), with the
 * backward of RoPE -- the rotation by the negative angle -- applied to dq and dk in the kernels' epilogues, in fp32,
 * before their one rounding (or before they are added to an fp32 accumulator: the rotation is linear).  dq and dk are
 * therefore gradients w.r.t. the UN-rotated q and k; no separate RoPE pass runs in the backward.  `out` is the bf16
 * forward output, `delta` an output as in pico_attn_bwd_fused; dq, dk and dv are all required.  dq_accumulate /
 * dkv_accumulate as in pico_attn_bwd (one block of a ring adds to the rank's running dq and to the chunk's travelling
 * dk / dv, context_parallel.py:85-106).  Positions: q_pos_offset + query row, k_pos_offset + key row (a ring block of
 * rank r over chunk c: r * Sc and c * Sc).
 */
int pico_attn_bwd_rope(const pico_attn_desc* desc, const void* q_rot, const void* k_rot, const void* v,
                       const void* dout, const void* out, const float* lse, float* delta,
                       void* dq, const int64_t* dq_stride, int dq_dtype, int dq_accumulate,
                       void* dk, void* dv, const int64_t* dkv_stride, int dkv_dtype, int dkv_accumulate,
                       const pico_rope_tables* rope, int q_pos_offset, int k_pos_offset, void* stream);

/* ------------------------------------------------------------------ all ring steps of one rank in one launch
 * replaces: the loops of RingAttentionFunc.forward / backward  context_parallel.py:30-45, :63-106  when the K / V
 *           chunks a rank would receive step by step are all in this GPU's memory already (virtual ranks).
 * K / V are `count` chunks of chunk_len keys each, given by their base pointers; every chunk is addressed with the
 * descriptor's k_stride / v_stride (and dkv_stride), desc->Sk must equal count * chunk_len, and with count > 1
 * chunk_len must be a multiple of 128 (otherwise PICO_ERR_SHAPE: run the ring step by step with pico_attn_fwd(merge)
 * / pico_attn_bwd(accumulate)).  Key j of the launch is row j % chunk_len of chunk j / chunk_len and sits at position
 * j: list the chunks in the order of their positions (for a causal ring: the chunks of ranks 0 .. r, q_offset =
 * r * chunk_len).  The online softmax runs across the chunks inside the kernel -- no per-step partial result, no
 * merge pass, no fp32 running out.
 * Backward: dk[c] / dv[c] receive chunk c's gradient; a NULL pair means that chunk's gradient is not wanted; bit c of
 * accumulate_mask adds to what is there (fp32 only: the chunk's travelling accumulators).
 * dk_final[c] / dv_final[c] (optional, given together): this launch holds the LAST block that chunk c's gradient is
 * waiting for (context_parallel.py:104-110: the accumulators have come round the ring).  The chunk's total -- what
 * dk[c] / dv[c] hold, if bit c of accumulate_mask is set, plus this launch's block -- is then rounded once and written
 * to dk_final[c] / dv_final[c] in bf16, addressed by final_stride (element strides b, h, s); dk[c] / dv[c] are only
 * read.  It saves the fp32 write, the read-back and the separate cast.
 */
#define PICO_MAX_KV_CHUNKS 16
typedef struct pico_kv_chunks {
  int32_t count;                       /* 1 .. PICO_MAX_KV_CHUNKS */
  int32_t chunk_len;
  const void* k[PICO_MAX_KV_CHUNKS];
  const void* v[PICO_MAX_KV_CHUNKS];
  void* dk[PICO_MAX_KV_CHUNKS];        /* backward only */
  void* dv[PICO_MAX_KV_CHUNKS];
  void* dk_final[PICO_MAX_KV_CHUNKS];  /* backward only, optional */
  void* dv_final[PICO_MAX_KV_CHUNKS];
  int64_t final_stride[3];
  uint32_t accumulate_mask;
  uint32_t reserved;
} pico_kv_chunks;

/* pico_attn_fwd over a chunk list.  rope = NULL: q and the chunks' k are used as they are.  rope != NULL: q is rotated
 * in the kernel as in pico_attn_fwd_rope (position q_pos_offset + row; the chunks' k must be rotated already) and
 * written to q_rot if that is given. */
int pico_attn_fwd_chunks(const pico_attn_desc* desc, const void* q, const pico_kv_chunks* kv, void* out, float* lse,
                         int out_dtype, int merge, const pico_rope_tables* rope, int q_pos_offset, void* q_rot,
                         const int64_t* q_rot_stride, void* stream);

/* pico_attn_bwd_fused over a chunk list.  `out` (forward output, dtype out_dtype, addressed like dout) may be NULL:
 * `delta` is then an input, otherwise it is written (by the dQ kernel's prologue when out is bf16 and dq is wanted, by
 * an internal pre-pass otherwise).  dq NULL: not wanted.  rope != NULL: q and the chunks' k are the rotated tensors and
 * dq / dk leave un-rotated as in pico_attn_bwd_rope (key position = k_pos_offset + key index of the launch). */
int pico_attn_bwd_chunks(const pico_attn_desc* desc, const void* q, const pico_kv_chunks* kv, const void* dout,
                         const void* out, int out_dtype, const float* lse, float* delta,
                         void* dq, const int64_t* dq_stride, int dq_dtype, int dq_accumulate,
                         const int64_t* dkv_stride, int dkv_dtype,
                         const pico_rope_tables* rope, int q_pos_offset, int k_pos_offset, void* stream);

/* fp32 -> bf16/fp32 conversion with layout change: src [B,H,S,D] contiguous fp32,
 * dst addressed by dst_stride (b,h,s).  Used to hand dq_acc back in the dtype / layout of q.
 * No counterpart in the reference (autograd does the cast, context_parallel.py:110).
 */
int pico_convert_f32(const float* src, void* dst, int64_t B, int64_t H, int64_t S, int64_t D,
                     int64_t dst_stride_b, int64_t dst_stride_h, int64_t dst_stride_s,
                     int dst_dtype, void* stream);

/* ------------------------------------------------------------------ loss
 * replaces: F.cross_entropy(outputs.view(S*B, V), target_ids, reduction='mean')  train.py:46-49  and its autograd.
 * logits: [rows, vocab] with row pitch ld (elements; a multiple of 8 for bf16, 4 for fp32), dtype `dtype`;
 * targets: [rows] int64, each in [0, vocab) or equal to ignore_index (torch's default is -100).  A target outside
 *          [0, vocab) that is not ignore_index is never used as an index: the row is treated as ignored (loss 0,
 *          gradient row 0) in both directions, where torch asserts on the device.
 * forward : loss[r] = logsumexp(logits[r]) - logits[r][target[r]] (0 for an ignored row) and lse[r], both fp32 [rows].
 *           The mean over the rows that are not ignored is left to the caller (one small reduction).
 * backward: dlogits[r][j] = (exp(logits[r][j] - lse[r]) - (j == target[r])) * scale[0], 0 for an ignored row;
 *           `scale` is a DEVICE pointer to one float (upstream gradient / number of rows that count), so no host
 *           synchronisation is needed; dlogits has pitch dld and may alias logits.
 */
int pico_cross_entropy_fwd(const void* logits, const int64_t* targets, float* loss, float* lse, int64_t rows,
                           int64_t vocab, int64_t ld, int64_t ignore_index, int dtype, void* stream);
int pico_cross_entropy_bwd(const void* logits, const int64_t* targets, const float* lse, const float* scale,
                           void* dlogits, int64_t rows, int64_t vocab, int64_t ld, int64_t dld, int64_t ignore_index,
                           int dtype, void* stream);

/* ------------------------------------------------------------------ optimizer step
 * replaces: torch.optim.AdamW(model.parameters(), lr).step()  train.py:204-209,240  for low-precision parameters
 *           with fp32 state: the reference keeps the AdamW state in the parameter dtype; here master weights and
 *           both moments are fp32 and the bf16 parameter is rewritten from the master weight in the same pass.
 * Same order of operations as torch's AdamW (decoupled weight decay, no amsgrad):
 *   p *= 1 - lr*wd;  m += (g - m)*(1 - beta1);  v = v*beta2 + g*g*(1 - beta2);
 *   p -= lr/bc1 * m / (sqrt(v)/sqrt(bc2) + eps),  bc_i = 1 - beta_i^step,  g = grad * grad_scale.
 * param_lp: [n] bf16, written (may be NULL); master, exp_avg, exp_avg_sq: [n] fp32, updated in place;
 * grad: [n] of grad_dtype (PICO_BF16 or PICO_F32); step counts from 1.
 */
int pico_adamw(void* param_lp, float* master, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
               int64_t n, float lr, float beta1, float beta2, float eps, float weight_decay, int64_t step,
               float grad_scale, void* stream);
/* The same step on the bf16 parameter itself, no master copy: param [n] of param_dtype (PICO_BF16) is read, updated
 * and rounded once in place.  exp_avg / exp_avg_sq are [n] of state_dtype:
 *   PICO_F32   fp32 moments ("bf16 parameters with fp32 AdamW state"), 22 bytes of traffic per parameter;
 *   PICO_BF16  the state as the reference holds it (train.py:209 builds AdamW on the bf16 parameters, so torch keeps
 *              exp_avg and exp_avg_sq in bf16), 14 bytes; fp32 arithmetic and one rounding per state, which is what
 *              torch's fused AdamW does (its default for-each path rounds after every operation).
 */
int pico_adamw_lp(void* param, const void* grad, int grad_dtype, void* exp_avg, void* exp_avg_sq, int64_t n,
                  int param_dtype, int state_dtype, float lr, float beta1, float beta2, float eps, float weight_decay,
                  int64_t step, float grad_scale, void* stream);
/* The step for `count` tensors at once (what torch's for-each / fused AdamW does for the whole parameter list of
 * train.py:209): host arrays of `count` device pointers and sizes; the library packs them into the arguments of as
 * few launches as they fit (48 tensors each), so a model's ~200 parameter tensors cost 5 launches instead of 200.
 * (weight_dtype, state_dtype) = (PICO_F32, PICO_F32): weights are the fp32 master weights and param_lps (the array
 * or single entries may be NULL) receive their bf16 copies, as pico_adamw; (PICO_BF16, PICO_F32 or PICO_BF16): weights
 * are the bf16 parameters themselves and param_lps must be NULL, as pico_adamw_lp.  All gradients share grad_dtype.
 * Tensors of size 0 are skipped.  Every tensor is checked before the first launch: a rejected call has changed nothing.
 */
int pico_adamw_multi(int count, void* const* weights, void* const* param_lps, const void* const* grads,
                     void* const* exp_avgs, void* const* exp_avg_sqs, const int64_t* sizes, int weight_dtype,
                     int state_dtype, int grad_dtype, float lr, float beta1, float beta2, float eps, float weight_decay,
                     int64_t step, float grad_scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PICOTRON_AMD_H */
