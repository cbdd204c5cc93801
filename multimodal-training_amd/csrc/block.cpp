// One transformer block of the vision tower behind a single C call each way: the fixed launch sequence of the block's
// forward and of its backward (Qwen2_5_VLVisionBlock.forward, modeling_qwen2_5_vl.py:776-792, with _forward_standard
// :385-472 and the MLP :203-204, and their autograd), issued from here instead of one host-language call per kernel.
// Nothing is computed here: every step is one of the library's own entry points with the operands the caller laid out,
// so the results are those of the same sequence issued call by call.  No allocation, no synchronisation; the only
// streams and events used are the caller's.
#include <math.h>
#include <string.h>

#include "mvit_common.h"

namespace {

constexpr int RMS_PARTIALS = 1024;  // work-groups (= partial rows) of the RMSNorm backward

struct Bump {  // hands out 256-byte aligned pieces of the caller's workspace
  char* base;
  int64_t used, size;
  void* take(int64_t bytes) {
    void* p = base ? base + used : nullptr;
    used += (bytes + 255) / 256 * 256;
    return p;
  }
};

inline int colsum_partials(int64_t rows) {
  const int64_t n = (rows + 15) / 16;
  return (int)(n < 1 ? 1 : (n > 64 ? 64 : n));
}

inline int64_t esize(int dtype) { return dtype == MVIT_BF16 ? 2 : 4; }

inline const char* at(const void* p, int64_t elems, int dtype) { return static_cast<const char*>(p) + elems * esize(dtype); }
inline char* at(void* p, int64_t elems, int dtype) { return static_cast<char*>(p) + elems * esize(dtype); }

mvit_gemm_args gemm_args(int dtype, int out_dtype) {
  mvit_gemm_args g;
  memset(&g, 0, sizeof(g));
  g.dtype = dtype;
  g.out_dtype = out_dtype;
  g.split_k = 1;
  return g;
}

// Layout of the backward's workspace; with base == nullptr only the size is computed.
struct BwdWorkspace {
  float *colsum, *swiglu_cols, *rms, *delta, *splitk;
  int64_t delta_elems, splitk_bytes, total;
};
BwdWorkspace plan_bwd_workspace(const mvit_block_args* a, void* base) {
  const int64_t S = a->S, C = a->C, I = a->I, Ipad = a->Ipad;
  Bump b{static_cast<char*>(base), 0, 0};
  BwdWorkspace w;
  w.colsum = static_cast<float*>(b.take(64 * 3 * C * 4));
  w.swiglu_cols = static_cast<float*>(b.take((S + 255) / 256 * 2 * Ipad * 4));
  w.rms = static_cast<float*>(b.take((int64_t)RMS_PARTIALS * C * 4));
  w.delta_elems = mvit_attn_bwd_delta_elems(a->max_seqlen, S, a->nheads, a->head_dim, a->dtype);
  w.delta = static_cast<float*>(b.take(w.delta_elems * 4));
  const int64_t sk[4] = {a->split_k_down * C * I, a->split_k_gate_up * 2 * Ipad * C, a->split_k_proj * C * C, a->split_k_qkv * 3 * C * C};
  w.splitk_bytes = 0;
  for (int64_t n : sk) w.splitk_bytes = n * 4 > w.splitk_bytes ? n * 4 : w.splitk_bytes;
  w.splitk = static_cast<float*>(b.take(w.splitk_bytes));
  w.total = b.used;
  return w;
}

int check_block(const char* who, const mvit_block_args* a) {
  MVIT_REQUIRE(a != nullptr, "%s: null arguments", who);
  MVIT_REQUIRE(a->dtype == MVIT_BF16 || a->dtype == MVIT_F32, "%s: dtype %d", who, a->dtype);
  MVIT_REQUIRE(a->S >= 0 && a->C > 0 && a->I > 0 && a->Ipad >= a->I && a->Ipad % 8 == 0 && a->nheads > 0 && a->head_dim > 0 &&
                   (int64_t)a->nheads * a->head_dim == a->C,
               "%s: bad sizes (S=%lld C=%d I=%d Ipad=%d heads=%d x %d)", who, (long long)a->S, a->C, a->I, a->Ipad, a->nheads, a->head_dim);
  MVIT_REQUIRE(a->norm1 && a->norm2 && a->wqkv && a->bqkv && a->wproj && a->bproj && a->wgu && a->bgu && a->wdown && a->bdown,
               "%s: null weight operand", who);
  MVIT_REQUIRE(a->cu && a->cos && a->sin && a->n_seg >= 0 && a->max_seqlen >= 0, "%s: attention geometry missing", who);
  MVIT_REQUIRE(a->x && a->n1 && a->rstd1 && a->qkv && a->o && a->lse && a->x1 && a->n2 && a->rstd2 && a->h, "%s: null activation buffer", who);
  return MVIT_OK;
}

}  // namespace

#define STEP(call)                \
  do {                            \
    if (int rc__ = (call)) return rc__; \
  } while (0)

extern "C" int mvit_block_fwd(const mvit_block_args* a, mvit_stream_t stream) {
  if (int rc = check_block("block_fwd", a)) return rc;
  if (a->S == 0) return MVIT_OK;
  const int dt = a->dtype;
  const int64_t S = a->S, C = a->C, Ipad = a->Ipad;
  const int H = a->nheads, hd = a->head_dim;

  STEP(mvit_rmsnorm_fwd(a->x, a->norm1, a->n1, a->rstd1, S, C, a->eps, dt, stream));
  {  // qkv = n1 . Wqkv^T + b
    mvit_gemm_args g = gemm_args(dt, dt);
    g.epilogue = MVIT_EPI_BIAS;
    g.M = S; g.N = 3 * C; g.K = C;
    g.A = a->n1; g.lda = C; g.B = a->wqkv; g.ldb = C; g.bias = a->bqkv; g.C = a->qkv; g.ldc = 3 * C;
    STEP(mvit_gemm(&g, stream));
  }
  // rotary embedding of q and k in place; the queries also take the softmax scale in base-2 units
  STEP(mvit_rope_scaled(a->qkv, a->cos, a->sin, S, 2 * H, hd, 3 * C, 0, H, a->q_lead_scale, dt, stream));
  if (!a->skip_attention)
    STEP(mvit_attn_fwd(a->qkv, at(a->qkv, C, dt), at(a->qkv, 2 * C, dt), a->o, a->lse, a->cu, a->seg_order, a->n_seg, a->max_seqlen, S, H, hd,
                       3 * C, 3 * C, 3 * C, C, a->attn_scale, dt, stream));
  {  // x1 = x + o . Wproj^T + b
    mvit_gemm_args g = gemm_args(dt, dt);
    g.epilogue = MVIT_EPI_BIAS_RES;
    g.M = S; g.N = C; g.K = C;
    g.A = a->o; g.lda = C; g.B = a->wproj; g.ldb = C; g.bias = a->bproj; g.C = a->x1; g.ldc = C; g.R = a->x; g.ldr = C;
    STEP(mvit_gemm(&g, stream));
  }
  STEP(mvit_rmsnorm_fwd(a->x1, a->norm2, a->n2, a->rstd2, S, C, a->eps, dt, stream));
  {  // h = silu(n2 . Wg^T + bg) * (n2 . Wu^T + bu); the pre-activations go to gu when the backward will want them
    mvit_gemm_args g = gemm_args(dt, dt);
    g.epilogue = MVIT_EPI_SWIGLU;
    g.M = S; g.N = Ipad; g.K = C;
    g.A = a->n2; g.lda = C; g.B = a->wgu; g.B2 = at(a->wgu, Ipad * C, dt); g.ldb = C;
    g.bias = a->bgu; g.bias2 = at(a->bgu, Ipad, dt);
    g.C = a->h; g.ldc = Ipad; g.aux = a->gu; g.ldaux = a->gu ? 2 * Ipad : 0; g.aux_off = Ipad;
    STEP(mvit_gemm(&g, stream));
  }
  if (a->x2) {  // x2 = x1 + h . Wdown^T + b
    mvit_gemm_args g = gemm_args(dt, dt);
    g.epilogue = MVIT_EPI_BIAS_RES;
    g.M = S; g.N = C; g.K = Ipad;
    g.A = a->h; g.lda = Ipad; g.B = a->wdown; g.ldb = Ipad; g.bias = a->bdown; g.C = a->x2; g.ldc = C; g.R = a->x1; g.ldr = C;
    STEP(mvit_gemm(&g, stream));
  }
  return MVIT_OK;
}

extern "C" int64_t mvit_block_bwd_workspace_bytes(const mvit_block_args* a) {
  if (a == nullptr) return 0;
  return plan_bwd_workspace(a, nullptr).total;
}

extern "C" int mvit_block_bwd(const mvit_block_args* a, mvit_stream_t stream) {
  if (int rc = check_block("block_bwd", a)) return rc;
  MVIT_REQUIRE(a->gu && a->dx2 && a->dx && a->dgu && a->dn && a->dx1 && a->dqkv, "block_bwd: null gradient buffer");
  MVIT_REQUIRE(a->g_norm1 && a->g_norm2 && a->g_wqkv && a->g_bqkv && a->g_wproj && a->g_bproj && a->g_wgu && a->g_bgu && a->g_wdown && a->g_bdown,
               "block_bwd: null parameter-gradient buffer");
  MVIT_REQUIRE(a->grad_dtype == MVIT_BF16 || a->grad_dtype == MVIT_F32, "block_bwd: grad_dtype %d", a->grad_dtype);
  MVIT_REQUIRE(a->split_k_down >= 1 && a->split_k_gate_up >= 1 && a->split_k_proj >= 1 && a->split_k_qkv >= 1, "block_bwd: split_k counts must be >= 1");
  const bool two = a->side_stream != nullptr;
  if (two) MVIT_REQUIRE(a->events[0] && a->events[1] && a->events[2] && a->events[3] && a->events[4], "block_bwd: a second stream needs five events");
  if (a->S == 0) return MVIT_OK;
  const BwdWorkspace w = plan_bwd_workspace(a, a->workspace);
  MVIT_REQUIRE(a->workspace && mvit_aligned16(a->workspace) && a->workspace_bytes >= w.total, "block_bwd: the workspace holds %lld bytes, %lld are needed",
               (long long)a->workspace_bytes, (long long)w.total);
  const int dt = a->dtype, gdt = a->grad_dtype;
  const int64_t S = a->S, C = a->C, I = a->I, Ipad = a->Ipad;
  const int H = a->nheads, hd = a->head_dim;
  hipStream_t main_s = reinterpret_cast<hipStream_t>(stream), side_s = reinterpret_cast<hipStream_t>(a->side_stream);

  // Weight and bias gradients feed nothing else in the block: with a second stream they start there once their inputs
  // are complete on the main stream (event n) and are joined at the end; without one they run in line.
  auto fork = [&](int n) -> mvit_stream_t {
    if (!two) return stream;
    hipEvent_t ev = reinterpret_cast<hipEvent_t>(a->events[n]);
    if (hipEventRecord(ev, main_s) != hipSuccess || hipStreamWaitEvent(side_s, ev, 0) != hipSuccess) {
      mvit_set_error(MVIT_ERR_LAUNCH, "block_bwd: event %d: %s", n, hipGetErrorString(hipGetLastError()));
      return nullptr;
    }
    return a->side_stream;
  };
  auto bias_grad = [&](const void* dy, int64_t ld, int64_t cols, void* out, mvit_stream_t st) -> int {
    const int np = colsum_partials(S);
    STEP(mvit_colsum(dy, ld, S, cols, w.colsum, np, dt, st));
    return mvit_reduce_partials(w.colsum, np, cols, out, gdt, st);
  };
  // dW[M, N] = dY^T . X over the S rows
  auto weight_grad = [&](const void* dy, int64_t ldy, int64_t M, const void* x, int64_t ldx, int64_t N, void* out, int split_k, mvit_stream_t st) -> int {
    mvit_gemm_args g = gemm_args(dt, gdt);
    g.trans_a = 1; g.trans_b = 1;
    g.M = M; g.N = N; g.K = S;
    g.A = dy; g.lda = ldy; g.B = x; g.ldb = ldx; g.C = out; g.ldc = N;
    if (split_k > 1) {
      g.split_k = split_k; g.workspace = w.splitk; g.workspace_bytes = (int64_t)split_k * M * N * 4;
    }
    return mvit_gemm(&g, st);
  };

  // ---- MLP: x2 = x1 + down(silu(g) * u)
  {
    mvit_stream_t st = fork(0);
    if (!st && two) return MVIT_ERR_LAUNCH;
    STEP(bias_grad(a->dx2, C, C, a->g_bdown, st));
    STEP(weight_grad(a->dx2, C, C, a->h, Ipad, I, a->g_wdown, a->split_k_down, st));
  }
  {  // dgu = (dx2 . Wdown) through the SwiGLU derivative; per-tile column sums of dgu come back with it
    mvit_gemm_args g = gemm_args(dt, dt);
    g.trans_b = 1; g.epilogue = MVIT_EPI_SWIGLU_BWD;
    g.M = S; g.N = Ipad; g.K = C;
    g.A = a->dx2; g.lda = C; g.B = a->wdown; g.ldb = Ipad; g.C = a->dgu; g.ldc = 2 * Ipad; g.R = a->gu; g.ldr = 2 * Ipad; g.aux_off = Ipad;
    g.workspace = w.swiglu_cols; g.workspace_bytes = (S + 255) / 256 * 2 * Ipad * 4;
    STEP(mvit_gemm(&g, stream));
  }
  {
    mvit_stream_t st = fork(1);
    if (!st && two) return MVIT_ERR_LAUNCH;
    STEP(mvit_reduce_partials(w.swiglu_cols, (int)((S + 255) / 256), 2 * Ipad, a->g_bgu, gdt, st));
    STEP(weight_grad(a->dgu, 2 * Ipad, 2 * Ipad, a->n2, C, C, a->g_wgu, a->split_k_gate_up, st));
  }
  {  // dn2 = dgu . Wgu
    mvit_gemm_args g = gemm_args(dt, dt);
    g.trans_b = 1;
    g.M = S; g.N = C; g.K = 2 * Ipad;
    g.A = a->dgu; g.lda = 2 * Ipad; g.B = a->wgu; g.ldb = C; g.C = a->dn; g.ldc = C;
    STEP(mvit_gemm(&g, stream));
  }
  STEP(mvit_rmsnorm_bwd(a->dn, a->x1, a->norm2, a->rstd2, a->dx2, a->dx1, w.rms, RMS_PARTIALS, S, C, dt, stream));
  STEP(mvit_reduce_partials(w.rms, RMS_PARTIALS, C, a->g_norm2, gdt, stream));

  // ---- attention: x1 = x + proj(attn(rope(qkv(norm1(x)))))
  {
    mvit_stream_t st = fork(2);
    if (!st && two) return MVIT_ERR_LAUNCH;
    STEP(bias_grad(a->dx1, C, C, a->g_bproj, st));
    STEP(weight_grad(a->dx1, C, C, a->o, C, C, a->g_wproj, a->split_k_proj, st));
  }
  {  // d_o = dx1 . Wproj  (into the dn buffer, whose contents the norm backward above has consumed)
    mvit_gemm_args g = gemm_args(dt, dt);
    g.trans_b = 1;
    g.M = S; g.N = C; g.K = C;
    g.A = a->dx1; g.lda = C; g.B = a->wproj; g.ldb = C; g.C = a->dn; g.ldc = C;
    STEP(mvit_gemm(&g, stream));
  }
  STEP(mvit_attn_bwd(a->qkv, at(a->qkv, C, dt), at(a->qkv, 2 * C, dt), a->o, a->dn, a->lse, a->dqkv, at(a->dqkv, C, dt), at(a->dqkv, 2 * C, dt),
                     w.delta, w.delta_elems, a->cu, a->seg_order, a->n_seg, a->max_seqlen, S, H, hd, 3 * C, 3 * C, 3 * C, C, C, 3 * C, 3 * C, 3 * C,
                     a->attn_scale, dt, stream));
  STEP(mvit_rope_scaled(a->dqkv, a->cos, a->sin, S, 2 * H, hd, 3 * C, 1, H, a->q_lead_scale, dt, stream));
  {
    mvit_stream_t st = fork(3);
    if (!st && two) return MVIT_ERR_LAUNCH;
    STEP(bias_grad(a->dqkv, 3 * C, 3 * C, a->g_bqkv, st));
    STEP(weight_grad(a->dqkv, 3 * C, 3 * C, a->n1, C, C, a->g_wqkv, a->split_k_qkv, st));
  }
  {  // dn1 = dqkv . Wqkv
    mvit_gemm_args g = gemm_args(dt, dt);
    g.trans_b = 1;
    g.M = S; g.N = C; g.K = 3 * C;
    g.A = a->dqkv; g.lda = 3 * C; g.B = a->wqkv; g.ldb = C; g.C = a->dn; g.ldc = C;
    STEP(mvit_gemm(&g, stream));
  }
  STEP(mvit_rmsnorm_bwd(a->dn, a->x, a->norm1, a->rstd1, a->dx1, a->dx, w.rms, RMS_PARTIALS, S, C, dt, stream));
  STEP(mvit_reduce_partials(w.rms, RMS_PARTIALS, C, a->g_norm1, gdt, stream));
  if (two) {  // the gradients are complete on the main stream when the call's work is
    hipEvent_t ev = reinterpret_cast<hipEvent_t>(a->events[4]);
    if (hipEventRecord(ev, side_s) != hipSuccess || hipStreamWaitEvent(main_s, ev, 0) != hipSuccess)
      return mvit_set_error(MVIT_ERR_LAUNCH, "block_bwd: joining the second stream: %s", hipGetErrorString(hipGetLastError()));
  }
  return MVIT_OK;
}
