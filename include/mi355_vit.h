/*
 * libmi355vit -- C ABI of the MI355X (gfx950) kernels behind the Qwen2.5-VL
 * vision-tower forward/backward.
 *
 * The reference (ray-project/multimodal-training) has no native boundary on
 * this path: every entry point below replaces a span of PyTorch/ATen calls in
 * the reference's Python, cited as file:line relative to the reference root
 * ("modeling" = python/models/qwen2_5_vl/modeling_qwen2_5_vl.py, "spu" =
 * python/models/qwen2_5_vl/sequence_parallel_utils.py, "[tf]" = transformers
 * models/qwen2/modeling_qwen2.py).
 *
 * Conventions
 *   - every function returns 0 on success or a negative MVIT_ERR_* code;
 *     mvit_last_error() then holds a message (thread-local);
 *   - nothing here allocates, frees or synchronises: the caller passes every
 *     output and workspace buffer and the HIP stream to enqueue on;
 *   - all pointers are device pointers unless the parameter says "host";
 *   - `dtype` is MVIT_F32 or MVIT_BF16 (storage type of activations/weights;
 *     accumulation is always fp32);
 *   - row-major everywhere; `ld*` / `*_stride` are in elements.
 */
#ifndef MI355_VIT_H
#define MI355_VIT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mvit_stream_t; /* hipStream_t */

enum { MVIT_F32 = 0, MVIT_BF16 = 1 };
enum { MVIT_OK = 0, MVIT_ERR_ARG = -1, MVIT_ERR_LAUNCH = -2, MVIT_ERR_UNSUPPORTED = -3 };

/* 200: mvit_attn_bwd takes the size of its workspace (delta_elems) and checks that outputs and inputs are disjoint;
 *      mvit_adam_tensor rows are 96 bytes (shadow copy fields).  A caller built against an older header must be
 *      rebuilt: compare mvit_version() with the value the header was written for. */
#define MVIT_VERSION 200
int mvit_version(void);
const char* mvit_last_error(void);

/* ---------------------------------------------------------------- host planners (integer, bit-exact) */

/* Position ids (h, w) of every patch in 2x2-merge-block order, repeated per frame.
 * Replaces rot_pos_emb's index construction, modeling:841-864.
 * grid_thw: host [n,3] int64; pos_ids: host [S,2] int64 with S = sum t*h*w. */
int mvit_rot_pos_ids(const int64_t* grid_thw, int64_t n, int merge, int64_t* pos_ids);

/* Window permutation of merged units and cumulative window lengths in patches with
 * consecutive duplicates removed.  Replaces get_window_index + unique_consecutive,
 * modeling:870-909 and :927-932.
 * window_index: host [S/merge^2] int64; cu_window: host int32 buffer of capacity cu_cap
 * (S/merge^2 + 1 always suffices); *n_cu receives the entry count. */
int mvit_window_index(const int64_t* grid_thw, int64_t n, int merge, int window_size, int patch_size,
                      int64_t* window_index, int32_t* cu_window, int64_t cu_cap, int64_t* n_cu);

/* cu_seqlens = [0, cumsum(repeat_interleave(h*w, t))], modeling:944-952.  cu: host int32 [sum t + 1]. */
int mvit_cu_seqlens(const int64_t* grid_thw, int64_t n, int32_t* cu, int64_t cu_cap, int64_t* n_cu);

/* Token-granular cut positions, spu:105-114.  cuts: host int64 [sp+1]. */
int mvit_sp_token_cuts(int64_t sample_len, int sp, int64_t* cuts);

/* Window-aligned cut positions, spu:117-164.  cut_pos, cut_idx: host int64 [sp+1]. */
int mvit_sp_window_cuts(int64_t sample_len, int sp, const int64_t* window_lengths, int64_t n_windows,
                        int64_t* cut_pos, int64_t* cut_idx);

/* ---------------------------------------------------------------- bandwidth-bound kernels */

/* y = w * cast(x_f32 * rsqrt(mean(x_f32^2) + eps)); rstd[rows] (fp32) is saved for the backward.
 * Replaces Qwen2RMSNorm.forward, [tf]:247-252 (call sites modeling:771-772, :253). */
int mvit_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t rows, int64_t cols,
                     float eps, int dtype, mvit_stream_t stream);

/* dx = [dx_add +] rstd * (dy*w - xhat * mean(dy*w*xhat)),  dw_partial[b, :] = sum over block b's rows of dy*xhat.
 * The autograd backward of the same lines.  dx_add may be null; dx may alias dx_add.
 * dw_partial: fp32 [n_partial, cols]; reduce it with mvit_reduce_partials. */
int mvit_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, const void* dx_add,
                     void* dx, float* dw_partial, int n_partial, int64_t rows, int64_t cols, int dtype,
                     mvit_stream_t stream);

/* out[c] = sum_b partial[b, c], written as `out_dtype`. */
int mvit_reduce_partials(const float* partial, int n_partial, int64_t cols, void* out, int out_dtype,
                         mvit_stream_t stream);

/* In-place rotary embedding of `nheads` heads of `head_dim` laid out at x[row*row_stride + h*head_dim + j]:
 *   out[j]        = x[j]*cos[j]               - x[j+half]*sin[j]
 *   out[j+half]   = x[j+half]*cos[j+half]     + x[j]*sin[j+half]
 * backward != 0 applies the transposed map (the gradient).  cos, sin: fp32 [rows, head_dim].
 * Replaces apply_rotary_pos_emb_vision / rotate_half, modeling:265-283. */
int mvit_rope(void* x, const float* cos, const float* sin, int64_t rows, int nheads, int head_dim,
              int64_t row_stride, int backward, int dtype, mvit_stream_t stream);

/* mvit_rope with the first `lead_heads` heads also multiplied by `lead_scale` before the single rounding to the storage
 * type (backward: after the transposed rotation).  The block passes its queries' softmax scale here
 * (head_dim^-1/2 * log2 e, the factor `q * scaling` of modeling:298-321 / the softmax_scale of the flash-attention call
 * :431-448 would apply) and calls the attention entry points with scale = 1 / log2 e: the scores then come from
 * once-rounded operands, as the reference's do. */
int mvit_rope_scaled(void* x, const float* cos, const float* sin, int64_t rows, int nheads, int head_dim,
                     int64_t row_stride, int backward, int lead_heads, float lead_scale, int dtype, mvit_stream_t stream);

/* dst[i, :] = src[index[i], :] for rows of row_bytes bytes (multiple of 2).  Bit-exact.
 * Replaces the window reorder x.view(M,4,C)[window_index] and its inverse, modeling:934-940, :1067-1068. */
int mvit_gather_rows(const void* src, const int64_t* index, void* dst, int64_t n_rows, int64_t row_bytes,
                     mvit_stream_t stream);

/* For each of nseg descriptors (src_row, dst_row, n_rows) (device int64 [nseg,3]) copy n_rows rows of
 * row_bytes bytes.  Bit-exact.  Replaces the torch.cat of slices in split_pack_by_sp (spu:265-269),
 * unpad_batch_to_pack (spu:342-346), build_local_rope (spu:395-404) and the re-interleave after the
 * ragged all-gather (modeling:1040-1064).  max_seg_rows bounds n_rows (grid sizing). */
int mvit_segment_copy(const void* src, void* dst, const int64_t* desc, int64_t nseg, int64_t max_seg_rows,
                      int64_t row_bytes, mvit_stream_t stream);

/* pack [sum len, row] -> padded [B, pad_len, row] filled with `pad_value` past each sample's length,
 * plus mask [B, pad_len] (uint8 0/1).  lens, offsets: device int64 [B].  elem_size 2 or 4; pad_bits is
 * the bit pattern of the pad value in that element type.  Replaces pad_pack_to_batch, spu:300-327. */
int mvit_pad_pack(const void* pack, void* padded, uint8_t* mask, const int64_t* lens, const int64_t* offsets,
                  int64_t batch, int64_t pad_len, int64_t row_elems, int elem_size, uint32_t pad_bits,
                  mvit_stream_t stream);

/* dst = cast(src) element-wise between MVIT_F32 and MVIT_BF16 over a [rows, cols] view with row strides. */
int mvit_cast2d(const void* src, int64_t src_ld, int src_dtype, void* dst, int64_t dst_ld, int dst_dtype,
                int64_t rows, int64_t cols, mvit_stream_t stream);

/* out[c] (+)= sum_r x[r, c]; fp32 partials [n_partial, cols], reduce with mvit_reduce_partials.
 * Bias gradients of the Linear layers (autograd of modeling:395-397, :471, :204, :255-257). */
int mvit_colsum(const void* x, int64_t ld, int64_t rows, int64_t cols, float* partial, int n_partial, int dtype,
                mvit_stream_t stream);

/* ---------------------------------------------------------------- MFMA GEMM with fused epilogues */

enum {
  MVIT_EPI_NONE = 0,       /* C = acc                                                         */
  MVIT_EPI_BIAS = 1,       /* C = acc + bias[n]                                               */
  MVIT_EPI_BIAS_RES = 2,   /* C = acc + bias[n] + R[m,n]                                      */
  MVIT_EPI_BIAS_GELU = 3,  /* aux = acc + bias[n];  C = gelu_erf(aux)                         */
  MVIT_EPI_SWIGLU = 4,     /* g = acc(B)+bias, u = acc(B2)+bias2; aux[m,n]=g, aux[m,aux_off+n]=u; C = silu(g)*u
                              (aux may be null: a forward that will not be differentiated gets C alone)  */
  MVIT_EPI_SWIGLU_BWD = 5, /* dh = acc; (g,u) = R[m,n], R[m,aux_off+n]; C[m,n]=dg, C[m,aux_off+n]=du */
  MVIT_EPI_GELU_BWD = 6,   /* C = acc * gelu_erf'(R[m,n])                                     */
  MVIT_EPI_ACCUM = 7       /* C = C + acc                                                     */
};

typedef struct mvit_gemm_args {
  int dtype;     /* of A, B, B2, R, aux */
  int out_dtype; /* of C */
  int trans_a;   /* 0: A is [M,K] (lda >= K);  1: A is [K,M] (lda >= M) */
  int trans_b;   /* 0: B is [N,K] (ldb >= K);  1: B is [K,N] (ldb >= N) */
  int epilogue;  /* MVIT_EPI_* */
  int64_t M, N, K;
  const void* A;
  int64_t lda;
  const void* B;
  const void* B2; /* SWIGLU only; same ldb */
  int64_t ldb;
  const void* bias;  /* [N], dtype; may be null for NONE/ACCUM/..._BWD */
  const void* bias2; /* SWIGLU only */
  void* C;
  int64_t ldc;
  const void* R; /* residual / saved pre-activation */
  int64_t ldr;
  void* aux;
  int64_t ldaux;
  int64_t aux_off; /* column offset of the second half in aux (SWIGLU) / R and C (SWIGLU_BWD) */
  void* workspace; /* split_k > 1: fp32 scratch of split_k * M * N floats.  MVIT_EPI_SWIGLU_BWD (optional): receives
                      fp32 column sums of C per 256-row tile, [ceil(M/256)][ldc] (columns [0,N) and
                      [aux_off, aux_off+N) are written); add the rows with mvit_reduce_partials for the bias gradient */
  int64_t workspace_bytes;
  int split_k;   /* <= 1: one work-group per tile walks all of K.  > 1 (EPI_NONE, EPI_BIAS, EPI_BIAS_RES): K is cut in
                    split_k slices whose fp32 partial tiles go to `workspace`; a second kernel sums them in a fixed
                    order and applies the epilogue (few output tiles, long contraction).  Available to any caller; the
                    vision tower uses it for weight gradients only, because a slice count chosen from M would make a
                    row's result depend on how many rows share its batch */
} mvit_gemm_args;

/* C[M,N] = epilogue(sum_k A[m,k] * B[n,k]).  Operands must be 16-byte aligned with lda/ldb multiples of
 * 16 bytes; K need not be a multiple of the tile (zero-filled).  Replaces nn.Linear / Conv3d(k==s) and
 * their autograd: modeling:230 (patch embed), :395-397 (q/k/v), :471 (proj), :204 (SwiGLU MLP), :261
 * (merger), with the element-wise ops of :204, :256, :784, :791 fused as epilogues. */
int mvit_gemm(const mvit_gemm_args* args, mvit_stream_t stream);

/* ---------------------------------------------------------------- varlen attention */

/* Per segment [cu[i], cu[i+1]) and head: O = softmax(Q K^T * scale) V, non-causal, fp32 softmax;
 * lse[h, s] = log sum exp of the scaled scores (fp32 [nheads, total]).
 * q/k/v/o element (s, h, j) lives at ptr[s*row_stride + h*head_dim + j].
 * Replaces the attention-backend call of _forward_standard, modeling:427-468 (eager: :298-321), and of
 * the sequence-parallel full-attention core, modeling:664-731 (nheads = heads / sp).
 * seg_order (device, n_seg entries, may be null): a permutation of 0..n_seg-1 giving the order in which the
 * segments are handed to the GPU.  Results do not depend on it; a work-group's run time grows with its
 * segment's length, so listing long segments first lets the short ones fill the tail of the launch. */
int mvit_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens,
                  const int32_t* seg_order, int n_seg, int max_seqlen, int64_t total, int nheads, int head_dim, int64_t q_stride,
                  int64_t k_stride, int64_t v_stride, int64_t o_stride, float scale, int dtype,
                  mvit_stream_t stream);

/* Gradients of the above.  delta: fp32 workspace of delta_elems floats; the call needs
 * mvit_attn_bwd_delta_elems(...) of them ([nheads, total] row sums of o * d_o, and for bf16 / head_dim 80 /
 * max_seqlen >= 512 two rescaled copies of the row statistics behind them) and refuses a shorter one.  dq/dk/dv use
 * the strides given and must not overlap any input (checked on the host, MVIT_ERR_ARG): the dq buffer is also used as
 * scratch (pre-scaled queries) before the result is written to it.
 * Replaces the autograd of the attention-backend call, modeling:427-468 and :664-731. */
int64_t mvit_attn_bwd_delta_elems(int max_seqlen, int64_t total, int nheads, int head_dim, int dtype);
int mvit_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                  void* dq, void* dk, void* dv, float* delta, int64_t delta_elems, const int32_t* cu_seqlens,
                  const int32_t* seg_order, int n_seg, int max_seqlen, int64_t total, int nheads, int head_dim, int64_t q_stride, int64_t k_stride,
                  int64_t v_stride, int64_t o_stride, int64_t do_stride, int64_t dq_stride, int64_t dk_stride,
                  int64_t dv_stride, float scale, int dtype, mvit_stream_t stream);

/* ---------------------------------------------------------------- one transformer block per call */

/* Operands of one block (Qwen2_5_VLVisionBlock.forward, modeling:776-792, with _forward_standard :385-472 and the MLP
 * :203-204) for mvit_block_fwd / mvit_block_bwd: the fixed launch sequence of the block behind one call each way, for
 * hosts whose per-call cost would otherwise exceed the kernels' run time at small batches.  Every step is one of the
 * entry points above on these operands, so the results are those of the same sequence issued call by call.
 * All tensors are contiguous, of `dtype` unless a float* says otherwise; all pointers are device pointers.
 *   weights  norm1, norm2 [C]; wqkv [3C, C], bqkv [3C] (q | k | v stacked); wproj [C, C], bproj [C];
 *            wgu [2*Ipad, C], bgu [2*Ipad] (gate rows [0, I), up rows [Ipad, Ipad+I), padding rows zero);
 *            wdown [C, Ipad] (padding columns zero), bdown [C]
 *   geometry cu / seg_order / n_seg / max_seqlen as for mvit_attn_fwd; cos, sin fp32 [S, head_dim];
 *            q_lead_scale = head_dim^-1/2 * log2 e applied to the queries in the rotary pass, attn_scale = 1 / log2 e
 *   forward  x [S,C] in; written: n1 [S,C], rstd1 [S], qkv [S,3C], o [S,C] and lse [nheads,S] (read instead when
 *            skip_attention != 0: the re-run of a checkpointed block that kept them), x1 [S,C], n2 [S,C], rstd2 [S],
 *            gu [S,2*Ipad] (null: not saved, for a forward that will not be differentiated), h [S,Ipad],
 *            x2 [S,C] (null: the down projection is skipped, for a re-run whose output nobody reads)
 *   backward reads x and everything the forward wrote (gu required) plus dx2 [S,C]; writes dx [S,C], the parameter
 *            gradients in `grad_dtype` laid out like the weights (g_wdown [C, I] without padding), and uses dgu
 *            [S,2*Ipad], dn [S,C], dx1 [S,C], dqkv [S,3C] and `workspace` (mvit_block_bwd_workspace_bytes) as scratch.
 *            split_k_*: K slices of the four weight-gradient GEMMs (>= 1).  side_stream (may be null): a second stream
 *            of the caller's on which weight and bias gradients run beside the input-gradient chain; it then needs
 *            five events of the caller's (hipEvent_t), and the call leaves the main stream waiting for the side one. */
typedef struct mvit_block_args {
  int dtype, grad_dtype;
  int C, I, Ipad, nheads, head_dim;
  int n_seg, max_seqlen, skip_attention;
  int split_k_down, split_k_gate_up, split_k_proj, split_k_qkv;
  float eps, q_lead_scale, attn_scale;
  int64_t S;
  const void *norm1, *norm2, *wqkv, *bqkv, *wproj, *bproj, *wgu, *bgu, *wdown, *bdown;
  const int32_t *cu, *seg_order;
  const float *cos, *sin;
  const void* x;
  void *n1, *qkv, *o, *x1, *n2, *gu, *h, *x2;
  float *rstd1, *rstd2, *lse;
  const void* dx2;
  void *dx, *dgu, *dn, *dx1, *dqkv;
  void *g_norm1, *g_norm2, *g_wqkv, *g_bqkv, *g_wproj, *g_bproj, *g_wgu, *g_bgu, *g_wdown, *g_bdown;
  void* workspace;
  int64_t workspace_bytes;
  mvit_stream_t side_stream;
  void* events[5];
} mvit_block_args;

int mvit_block_fwd(const mvit_block_args* args, mvit_stream_t stream);
int64_t mvit_block_bwd_workspace_bytes(const mvit_block_args* args);
int mvit_block_bwd(const mvit_block_args* args, mvit_stream_t stream);

/* ---------------------------------------------------------------- vision -> text hand-off */

/* Ranks the image placeholders of a token sequence: rank[t] = k (0-based) if input_ids[t] is the k-th entry equal
 * to image_token_id, else -1; positions[k] = t; counts[0] = number of placeholders; counts[1] = number of
 * placeholders whose label differs from ignore_label (0 when labels is null).  All device pointers; rank
 * [n_tokens] int32, positions [n_tokens] int64 (first counts[0] entries written), counts [2] int64.
 * Replaces the mask building and the counting guards of TextTrainer's forward, python/ray/text.py:883-910. */
int mvit_image_token_ranks(const int64_t* input_ids, const int64_t* labels, int64_t n_tokens, int64_t image_token_id,
                           int64_t ignore_label, int32_t* rank, int64_t* positions, int64_t* counts,
                           mvit_stream_t stream);

/* merged[t, :] = rank[t] >= 0 ? vision[rank[t], :] : embeds[t, :] over rows of row_bytes bytes (bit-exact copy);
 * with vision == NULL the selected rows are zero-filled instead.  A rank >= n_vision keeps the embeds row.
 * Forward: inputs_embeds.masked_scatter(image_mask, vision_embeds_flat), python/ray/text.py:913.  Backward: the
 * gradient of the text rows is mvit_merge_rows(grad, NULL, ...) and the gradient handed back to the vision actor
 * (text.py:1000-1019) is mvit_gather_rows(grad, positions, ...). */
int mvit_merge_rows(const void* embeds, const void* vision, const int32_t* rank, void* merged, int64_t n_tokens,
                    int64_t n_vision, int64_t row_bytes, mvit_stream_t stream);

/* ---------------------------------------------------------------- optimizer step (multi-tensor) */

#define MVIT_ADAM_CHUNK 8192 /* elements per work-group; a chunk never spans two tensors */

/* One parameter tensor of a multi-tensor launch.  The table lives in DEVICE memory and has n_tensors + 1
 * entries: entry i covers chunks [first_chunk(i), first_chunk(i+1)), first_chunk(i+1) - first_chunk(i) =
 * ceil(numel(i) / MVIT_ADAM_CHUNK), first_chunk(0) = 0, and the last entry is a sentinel whose first_chunk
 * is the total chunk count (its other fields are ignored).  The kernels trust the table.
 * step_size = lr / (1 - beta1^step) and bias_correction2_sqrt = sqrt(1 - beta2^step) are computed by the
 * caller in double precision, as torch/optim/adam.py does on the host. */
typedef struct {
  void* param;       /* [numel] dtype, updated in place */
  void* grad;        /* [numel] dtype; rewritten with grad * grad_scale when write_grad != 0 */
  void* exp_avg;     /* [numel] dtype, first moment */
  void* exp_avg_sq;  /* [numel] dtype, second moment */
  int64_t numel;
  int64_t first_chunk;
  float step_size;
  float bias_correction2_sqrt;
  float weight_decay; /* L2 term: grad + weight_decay * param, as torch.optim.Adam (not decoupled) */
  float unused;
  /* Optional second destination of the updated parameter (NULL: none): the operand copy the GEMMs read (a fused
   * q|k|v or gate|up weight, a weight with padded rows, a bf16 copy of an fp32 master weight).  The parameter is
   * seen as rows of shadow_cols elements and element (row, col) is also stored at shadow[row * shadow_ld + col]
   * (shadow_cols == 0: one row, i.e. a plain copy).  shadow_dtype is `dtype` or MVIT_BF16.  Only mvit_adam_step
   * reads these fields. */
  void* shadow;
  int64_t shadow_cols, shadow_ld;
  int32_t shadow_dtype, unused2;
} mvit_adam_tensor;

/* torch.optim.Adam(foreach=False, amsgrad=False, maximize=False) for every tensor of the table in one launch:
 *   g = grad * grad_scale; g += weight_decay * p; m += (1 - beta1) (g - m); v = v beta2 + (1 - beta2) g g;
 *   p -= step_size * m / (sqrt(v) / bias_correction2_sqrt + eps)
 * one operation at a time in fp32, each result rounded to `dtype` when that is bf16 (what the per-tensor
 * torch kernels do).  grad_scale is the clipping coefficient of Trainer._clip_gradients (1 = none); with
 * write_grad the scaled gradient is stored back, as the reference's in-place grad.mul_ leaves it.
 * The hyper-parameters are doubles (Python floats): 1 - beta1 and 1 - beta2 are formed in double and rounded
 * to fp32 once, as they reach torch's kernels.
 * Replaces Trainer.optimizer_step -> self.optimizer.step() (trainer.py:158-189, optimizer built at :479-577)
 * and the scaling loop of Trainer._clip_gradients (trainer.py:123-156). */
int mvit_adam_step(const mvit_adam_tensor* tensors, int n_tensors, int64_t n_chunks, double beta1, double beta2,
                   double eps, double grad_scale, int write_grad, int dtype, mvit_stream_t stream);

/* out[0] (fp64, device) = sum over all tensors of the table of sum(grad^2): only `grad`, `numel` and
 * `first_chunk` of each entry are read.  partial: fp32 workspace [n_chunks].  Replaces the per-tensor
 * norm(2).item() ** 2 loop of Trainer._compute_grad_norm_squared (trainer.py:293-308) with two launches
 * and one read-back by the caller. */
int mvit_grad_sumsq(const mvit_adam_tensor* tensors, int n_tensors, int64_t n_chunks, float* partial, double* out,
                    int dtype, mvit_stream_t stream);

/* mvit_grad_sumsq without the workspace argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight loops, harnesses that forbid hipMalloc): the per-chunk partial sums live in an array
 * built into the library (MVIT_SUMSQ_STATIC_MAX_CHUNKS floats = 1 MiB per GPU, held until the process ends).  It
 * has no counterpart in the reference.  Same results as mvit_grad_sumsq, bit for bit.  n_chunks above the maximum
 * is rejected with MVIT_ERR_ARG.  The first call on a device looks up the array's address (no allocation); no call
 * allocates or frees memory.  All calls on one GPU share the array: calls that overlap in time on one GPU (two
 * streams, two threads) race and must be serialised by the caller. */
#define MVIT_SUMSQ_STATIC_MAX_CHUNKS 262144 /* x MVIT_ADAM_CHUNK = 2^31 elements */
int mvit_grad_sumsq_static(const mvit_adam_tensor* tensors, int n_tensors, int64_t n_chunks, double* out, int dtype,
                           mvit_stream_t stream);

/* ---------------------------------------------------------------- input side: decoded frames -> pixel_values */

#define MVIT_PIXEL_ROW 1176 /* 3 channels x 2 frames x 14 x 14: one row of pixel_values */

/* One image or video of the batch: `frames` decoded RGB frames of height x width pixels, uint8, [frames][height]
 * [width][3] contiguous in device memory, already resized (height and width multiples of 28).  first_row is the
 * row of pixel_values its first patch goes to: the running sum of ceil(frames / 2) * (height / 14) * (width / 14).
 * The table has n_images + 1 entries; the last one only carries first_row = total number of rows. */
typedef struct mvit_image {
  const uint8_t* pixels;
  int32_t frames, height, width, reserved;
  int64_t first_row;
} mvit_image;

/* pixel_values[first_row + r, :] for every image of the table, in one launch:
 *   value = ((float)((double)byte * rescale) - mean[c]) / std[c]        (float32, then rounded to `dtype`)
 * rows in the order (temporal pair, 2x2 merge block row, merge block column, row in block, column in block),
 * columns in the order (channel, frame of the pair, y in patch, x in patch); a frame count that is odd is filled
 * up by using the last frame twice (a still image fills both halves of its rows).  `images` is a device pointer,
 * out is [total_rows, 1176] of dtype MVIT_F32 or MVIT_BF16.
 * Replaces the rescale / normalise / patchify steps of the image processor that the reference runs on CPU
 * workers through processor.apply_chat_template (python/data/preprocessing.py:134; transformers 4.57.0,
 * Qwen2VLImageProcessor._preprocess) and the concatenation of python/data/collator.py:134-156; the cast to the
 * model dtype is the one of the tower's first line (modeling_qwen2_5_vl.py, patch_embed input). */
int mvit_patchify(const mvit_image* images, int n_images, int64_t total_rows, void* out, double rescale, float mean_r,
                  float mean_g, float mean_b, float std_r, float std_g, float std_b, int dtype, mvit_stream_t stream);

/* The patch embedding straight from decoded frames: out[r, :] = row r of pixel_values (exactly the bf16 rows that
 * mvit_patchify makes for the same table and constants) x weight^T, bf16 MFMA with fp32 accumulation, without the
 * [total_rows, 1176] matrix ever being written.  The kernel contracts along memory (frame of the pair, y | x, channel)
 * instead of (channel, frame, y, x), so it takes the weight re-ordered by mvit_patch_embed_pack_weight:
 *   packed[n, (frame * 14 + y) * 48 + x * 3 + channel] = w[n, channel * 392 + frame * 196 + y * 14 + x], zero elsewhere;
 *   packed is [n_out, 1344] bf16, 16-byte aligned; w is [n_out, >= 1176] of dtype MVIT_BF16 or MVIT_F32, row pitch ldw.
 * Frame buffers must be 4-byte aligned (their size always is a multiple of 4: widths are multiples of 28); the table
 * is trusted as in mvit_patchify.  Rescale and normalisation run as one fused multiply-add per byte; constants for
 * which that does not reproduce mvit_patchify's bf16 values for all 3 x 256 inputs are rejected with
 * MVIT_ERR_UNSUPPORTED (the caller then uses mvit_patchify + mvit_gemm).  out is [total_rows, ldo >= n_out] of
 * out_dtype MVIT_BF16 or MVIT_F32.
 * Replaces the image processor's rescale / normalise / patchify (python/data/preprocessing.py:134) together with the
 * tower's patch embedding, Qwen2_5_VisionPatchEmbed.forward (python/models/qwen2_5_vl/modeling_qwen2_5_vl.py:225-231:
 * a Conv3d without bias whose kernel equals its stride, i.e. this matrix product). */
int mvit_patch_embed_pack_weight(const void* w, int dtype, int64_t ldw, int64_t n_out, void* packed, mvit_stream_t stream);
int mvit_patch_embed_frames(const mvit_image* images, int n_images, int64_t total_rows, const void* packed_w, int64_t n_out,
                            void* out, int64_t ldo, int out_dtype, double rescale, float mean_r, float mean_g, float mean_b,
                            float std_r, float std_g, float std_b, mvit_stream_t stream);

/* One resampling pass of PIL.Image.resize for 8-bit images along the middle axis of a contiguous uint8 array
 * [outer][in_len][inner] -> [outer][out_len][inner] (device memory): for output coordinate x the in-range window of
 * bounds[2x + 1] input coordinates starting at bounds[2x], weighted by the 22-bit fixed-point coefficients
 * kk[x * ksize + i]; accumulator = 2^21 + sum byte * weight, result = clamp(accumulator >> 22, 0, 255): Pillow's
 * libImaging/Resample.c (ImagingResampleHorizontal_8bpc / ImagingResampleVertical_8bpc), bit for bit.  A resize is
 * the horizontal pass (outer = frames * height, inner = 3) into an intermediate image followed by the vertical pass
 * (outer = frames, inner = new_width * 3); a pass whose size does not change is skipped by the caller.  bounds and kk
 * are device arrays that the host computes once per (in_len, out_len, filter) as Resample.c precompute_coeffs +
 * normalize_coeffs_8bpc do (Python: mi355_vit.pixels.resample_coefficients).  Contract for tables of the caller's
 * own: 0 <= bounds[2x], 0 <= bounds[2x + 1] <= ksize and bounds[2x] + bounds[2x + 1] <= in_len for every x; the device
 * arrays are not read back to check it, the kernels force every window into that range instead.
 * Replaces, for frames that are already on the GPU, the two PIL resizes in front of the patch rows: the reference's
 * own fixed-size BILINEAR resize (python/data/preprocessing.py:126-131) and the BICUBIC resize to the smart_resize
 * target inside the image processor (transformers 4.57.0 Qwen2VLImageProcessor, reached through
 * processor.apply_chat_template, python/data/preprocessing.py:134). */
int mvit_resample_u8(const uint8_t* src, uint8_t* dst, int64_t outer, int64_t in_len, int64_t out_len, int64_t inner,
                     const int32_t* bounds, const int32_t* kk, int ksize, mvit_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_VIT_H */
