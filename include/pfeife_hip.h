/*
 * pfeife_hip.h -- C ABI of libpfeife_hip.so: the gfx950 (MI355X) kernels behind
 * the pipeline-stage hot path of Pfeife.
 *
 * The reference (MerHS/pfeife) is pure Python and has no FFI of its own: every
 * device operation on its hot path is an ATen eager kernel reached through
 * `self.mods[node.idx](*inputs)` (pfeife/mp/worker.py:1494), through
 * `torch.autograd.backward` (pfeife/mp/worker.py:1585-1587), through the
 * same-rank handoff copies (pfeife/mp/worker.py:1096-1151) and through the
 * loss modules (pfeife/loss.py:53-70).  Each entry point below names the ATen
 * call site(s) of the reference that it replaces.
 *
 * Conventions
 *   - plain pointers and sizes only; all pointers are DEVICE pointers owned by
 *     the caller (PyTorch owns every buffer; nothing here allocates or frees);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *   - every call only enqueues work (no host synchronisation) and returns
 *     PF_OK (0) or a negative pf_status; pf_last_error() gives the text of the
 *     last failure on the calling thread;
 *   - sizes are in ELEMENTS unless a name says bytes; leading dimensions (ld*)
 *     are row strides in elements;
 *   - 16-bit operands of the vectorised kernels must be 16-byte aligned and have
 *     leading dimensions that are multiples of 8 elements (checked, PF_ERR_INVALID).
 */
#ifndef PFEIFE_HIP_H_
#define PFEIFE_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum pf_dtype { PF_F32 = 0, PF_F16 = 1, PF_BF16 = 2, PF_I64 = 3, PF_I32 = 4, PF_U8 = 5 };
enum pf_status { PF_OK = 0, PF_ERR_INVALID = -1, PF_ERR_UNSUPPORTED = -2, PF_ERR_HIP = -3 };
enum pf_act { PF_ACT_NONE = 0, PF_ACT_GELU = 1, PF_ACT_GELU_TANH = 2, PF_ACT_SILU = 3, PF_ACT_RELU = 4 };

/* ---- library state ------------------------------------------------------- */

/* ABI version of this header (bumped when a signature changes). */
int pf_version(void);
/* Text of the last error raised on the calling host thread ("" if none). */
const char* pf_last_error(void);
/* Checks that `device` is a gfx950 part and makes it current for the calling
 * thread.  Counterpart of torch.cuda.set_device in PfeifeState.__init__
 * (pfeife/mp/net_states.py:131-132). */
int pf_init(int device);

/* ---- launch-list replay -------------------------------------------------------------
 * The job loop of a step (pfeife/mp/worker.py:912-1006) issues the same kernels on the same
 * buffers every step.  Bracket one job's launches (ordinary calls of the entry points
 * below, on `stream`) with capture_begin / capture_end to obtain a hipGraphExec handle;
 * pf_graph_launch replays it with one host call.  `stream` must be a created stream (not
 * the legacy default stream).  No hipMemset nodes are ever recorded: every clear in this
 * library is a fill kernel. */
int pf_graph_capture_begin(void* stream);
int pf_graph_capture_end(void* stream, void** graph_exec_out);
int pf_graph_launch(void* graph_exec, void* stream);
int pf_graph_destroy(void* graph_exec);

/* ---- dense contractions (MFMA) -------------------------------------------
 * One descriptor covers every matrix product a stage executes:
 *   C[z] = epilogue( alpha * op(A[z]) . op(B[z]) )        for z in [0, batch1*batch2)
 * with the reduction over K, op(A) an M x K matrix and op(B) a K x N matrix.
 *   a_trans = 0 : A is stored M x K (element (m,k) at A[m*lda + k])
 *   a_trans = 1 : A is stored K x M (element (m,k) at A[k*lda + m])
 *   b_trans = 0 : B is stored N x K (element (k,n) at B[n*ldb + k])  -- an nn.Linear weight
 *   b_trans = 1 : B is stored K x N (element (k,n) at B[k*ldb + n])
 * so that  y = x W^T        is (a_trans 0, b_trans 0)   [F.linear forward]
 *          dx = dy W        is (a_trans 0, b_trans 1)   [grad wrt input]
 *          dW = dy^T x      is (a_trans 1, b_trans 1)   [grad wrt weight, beta = 1
 *                                                        accumulates into param.grad]
 * Batch z decomposes as z1 = z / batch2, z2 = z % batch2 and each operand moves
 * by  z1*stride1 + z2*stride2  elements (attention heads inside a packed qkv).
 *
 * Epilogue, applied per element v = alpha*acc in this order:
 *   v += bias[n]                       if bias
 *   v  = round_to(in_dtype, v)         if round_mid (mirrors autocast's 16-bit result)
 *   aux_out[m*ld_aux_out+n] = v        if aux_out   (kept for the backward pass; dtype = in_dtype)
 *   v  = act(v)                        if act != PF_ACT_NONE
 *   v *= act'(aux_in[m*ld_aux_in+n])   if dact != PF_ACT_NONE (dtype of aux_in = in_dtype)
 *   v += residual[m*ld_res+n]          if residual
 *   v += C[m*ldc+n]                    if beta == 1
 *   C[m*ldc+n] = v  (stored as c_dtype)
 * bias/aux/residual require batch1*batch2 == 1.
 *
 * in_dtype PF_F16/PF_BF16 run on v_mfma_f32_32x32x16 with fp32 accumulation;
 * in_dtype PF_F32 runs a full-precision fp32 FMA kernel (the fp32 parity path).
 * 16-bit products whose operands are both reduction-contiguous (a_trans = b_trans = 0,
 * K a multiple of 64) or both reduction-strided (a_trans = b_trans = 1) take the
 * direct-to-LDS kernel (tiles stream global -> LDS without staging registers, 3-5 stages
 * deep; transposing LDS reads for the strided case); every other 16-bit product takes a
 * register-staged kernel.
 *
 * Replaces: aten::linear / aten::addmm / aten::mm / aten::bmm forward and
 * backward, the autocast casts around them, aten::gelu(+backward), the
 * residual aten::add and autograd's AccumulateGrad add_ for weight gradients,
 * as executed by pfeife/mp/worker.py:1494 (forward) and :1585-1587 (backward).
 */
typedef struct pf_gemm_desc {
  int32_t in_dtype;
  int32_t c_dtype;
  int32_t a_trans;
  int32_t b_trans;
  int64_t M, N, K;
  const void* A;
  int64_t lda;
  const void* B;
  int64_t ldb;
  void* C;
  int64_t ldc;
  int64_t batch1, batch2;
  int64_t a_stride1, a_stride2;
  int64_t b_stride1, b_stride2;
  int64_t c_stride1, c_stride2;
  float alpha;
  int32_t beta;
  const void* bias;
  int32_t bias_dtype;
  int32_t round_mid;
  void* aux_out;
  int64_t ld_aux_out;
  int32_t act;
  int32_t dact;
  const void* aux_in;
  int64_t ld_aux_in;
  const void* residual;
  int64_t ld_res;
  int32_t res_dtype;
  int32_t variant; /* 0: automatic tile choice; otherwise one kernel variant by id (tuning
                      harnesses): 1..4 direct-to-LDS kernel with 256x256 / 256x128 / 128x128 /
                      192x256 tiles shared by four wavefronts, 5 / 6 its 128x128 / 256x128 tiles
                      with eight wavefronts as two grids that split each tile step's reduction
                      depth, 7 / 8 / 9 its 256x256 / 128x128 / 256x128 tiles with eight
                      wavefronts side by side, 11..14 register-staged kernel with 128x128 (8 wavefronts),
                      128x128, 128x64, 64x64 tiles; PF_ERR_INVALID if it cannot run the problem */
  float* colsum_ws; /* optional, with dact on the direct-to-LDS kernel (pf_gemm_variant ends in ", 5>"): the
                       launch also leaves the column sums of the 16-bit values it stores in C as partial
                       rows, ws[tile_row * N + column] for tile_row < ceil(M / BM) (BM: the variant's first
                       tile dimension): the bias gradient of the layer whose pre-activation gradient C is
                       (aten.sum of the reference's autograd, pfeife/mp/worker.py:1585-1587), finished by
                       pf_colreduce_finalize(_batch).  PF_ERR_UNSUPPORTED on any other kernel path. */
  const float* unscale_by; /* optional: device pointer to a loss scale s > 0, read when the kernel runs: the
                       product is multiplied by alpha / s[0] instead of alpha, so a gradient computed from a scaled
                       loss leaves the product unscaled (GradScaler.unscale_ of pfeife/mp/worker.py:1432-1436 without
                       a pass of its own) */
  float* nonfinite_flag; /* optional: set to 1.0f when a value written to C is not finite (the overflow check of
                       the same unscale_); only on the fp32-store / fp32-accumulate classes of the direct-to-LDS
                       kernel (pf_gemm_variant ends in ", 1>" or ", 4>"), PF_ERR_UNSUPPORTED elsewhere */
} pf_gemm_desc;

int pf_gemm(const pf_gemm_desc* desc, void* stream);
#define PF_GEMM_GROUP_MAX 8
/* n products in as few launches as possible.  Runs of consecutive descriptors that are weight
 * gradients (a_trans = b_trans = 1, 16-bit operands, fp32 C stored or accumulated, no epilogue operands,
 * no batch) and resolve to the same kernel instantiation share ONE launch (up to PF_GEMM_GROUP_MAX
 * per launch):
 * dW of a 1024x1024 weight covers only 64 of the 256 CUs on its own.  Everything else is issued
 * as by pf_gemm, in order.  The products of one call must not depend on each other's results.
 * torch.autograd issues the same products one by one (pfeife/mp/worker.py:1585-1587). */
int pf_gemm_grouped(const pf_gemm_desc* descs, int n, void* stream);
/* Measurement aid, no counterpart in the reference: `workgroups` workgroups of 4 wavefronts each issue
 * iters * 16 v_mfma_f32_32x32x16 instructions (2 * 32 * 32 * 16 FLOP each) on register-resident
 * fragments taken from `operands` (8 KiB of 16-bit values: 4 A fragments of 64 lanes x 8 values, then
 * 4 B fragments), with no loads, LDS traffic or barriers in the loop: the rate the matrix pipes
 * sustain under the board's power limit, the ceiling of any GEMM K loop.  sink: 256 * workgroups floats (per-lane checksums). */
int pf_mfma_rate(int dtype, const void* operands, int64_t iters, int workgroups, float* sink, void* stream);
/* Name of the kernel instantiation pf_gemm would launch for `desc`, spelled the
 * way a profiler prints it, e.g. "gemm16x_kernel<1, 256, 256, 32, 2, 4, 1, 5, false, false, 0>"
 * (dtype, tile M, tile N, stage depth, wavefront rows, columns, reduction split, stages, a_trans,
 * b_trans, epilogue class) or "gemm16_kernel<1, 128, 64, 64, 2, 2, false, true>".  Lets a harness attribute
 * measured kernel time to problem shapes.  No counterpart in the reference. */
int pf_gemm_variant(const pf_gemm_desc* desc, char* out, int cap);

/* ---- normalisation (HBM-bound, one wavefront per row) ---------------------
 * LayerNorm over the last dimension d of a [rows, d] matrix; gamma/beta are
 * fp32 [d] (beta may be NULL); mean/rstd are fp32 [rows] saved for backward.
 * Replaces aten::native_layer_norm / native_layer_norm_backward (stage
 * forward/backward, pfeife/mp/worker.py:1494, :1585-1587). */
int pf_layernorm_fwd(const void* x, int x_dtype, const float* gamma, const float* beta, void* y, int y_dtype,
                     float* mean, float* rstd, int64_t rows, int64_t d, float eps, void* stream);
/* dx = LN'(dy) (+ dx_add if given: the gradient already accumulated on x from
 * its other consumer, i.e. the residual branch); dgamma_acc/dbeta_acc (fp32
 * [d], may be NULL) are ACCUMULATED (+=), which is AccumulateGrad for the
 * norm's parameters.  workspace: >= pf_colreduce_workspace(rows, d) floats. */
int pf_layernorm_bwd(const void* dy, int dy_dtype, const void* x, int x_dtype, const float* gamma,
                     const float* mean, const float* rstd, const void* dx_add, int add_dtype, void* dx,
                     int dx_dtype, float* dgamma_acc, float* dbeta_acc, float* workspace, int64_t rows,
                     int64_t d, int defer_reduce, void* stream);
/* Normalisation backward with the follow-up work of a transformer block folded in.  Besides
 * dx (as above, + dx_add) it can write dx_lp, a second copy of dx in fp16/bf16: the form in
 * which the matrix products of the preceding layer read this gradient (torch autocast makes
 * that copy with a separate aten::_to_copy).  With want_colsum it also leaves the column
 * sums of dx_lp, i.e. the bias gradient of the linear layer whose output (+ residual) was
 * normalised (aten::sum in linear's backward).  mean == NULL selects RMSNorm.  Parameter
 * gradients and column sums are left as per-workgroup partial rows for
 * pf_colreduce_finalize_batch: workspace holds pf_norm_bwd_partials(rows) rows of
 * (want_colsum ? 3 : 2) * d floats, laid out [dgamma | dbeta | colsum].  want_colsum needs
 * 16-byte aligned operands, d % 8 == 0 and d <= 2048 (PF_ERR_UNSUPPORTED otherwise). */
typedef struct pf_norm_bwd_desc {
  const void* dy; const void* x; const float* gamma; const float* mean; const float* rstd;
  const void* dx_add; void* dx; void* dx_lp; float* workspace;
  int64_t rows, d;
  int32_t dy_dtype, x_dtype, add_dtype, dx_dtype, dx_lp_dtype, want_wgrad, want_colsum, reserved;
} pf_norm_bwd_desc;
int pf_norm_bwd_fused(const pf_norm_bwd_desc* desc, void* stream);
/* RMSNorm: y = x * rsqrt(mean(x^2) + eps) * gamma.  rstd fp32 [rows].
 * Replaces the pow/mean/rsqrt/mul chain (or aten::rms_norm) of Llama-style blocks. */
int pf_rmsnorm_fwd(const void* x, int x_dtype, const float* gamma, void* y, int y_dtype, float* rstd,
                   int64_t rows, int64_t d, float eps, void* stream);
int pf_rmsnorm_bwd(const void* dy, int dy_dtype, const void* x, int x_dtype, const float* gamma,
                   const float* rstd, const void* dx_add, int add_dtype, void* dx, int dx_dtype,
                   float* dgamma_acc, float* workspace, int64_t rows, int64_t d, int defer_reduce, void* stream);
/* GroupNorm over channels-last [B, HW, C] tensors (the memory layout this library keeps
 * convolutional feature maps in), `groups` groups of C/groups adjacent channels.
 * mean/rstd: fp32 [B*groups].  Backward: dx, and dgamma/dbeta ACCUMULATED (or, with
 * defer_reduce, left as per-sample partial rows [B][2][C] at the start of `workspace` for
 * pf_colreduce_finalize_batch: n_partials = B, stride = 2*C).  workspace holds
 * pf_groupnorm_workspace(B, C, groups) floats; C/groups <= 64 for the backward.
 * Replaces aten::native_group_norm(+backward) of the UNet stage
 * (bench_models/models/train_sdxl.py, diffusers ResnetBlock2D / Transformer2DModel). */
int pf_groupnorm_fwd(const void* x, int x_dtype, const float* gamma, const float* beta, void* y, int y_dtype,
                     float* mean, float* rstd, int64_t B, int64_t HW, int64_t C, int groups, float eps, void* stream);
int pf_groupnorm_bwd(const void* dy, int dy_dtype, const void* x, int x_dtype, const float* gamma, const float* mean,
                     const float* rstd, void* dx, int dx_dtype, float* dgamma_acc, float* dbeta_acc, float* workspace,
                     int64_t B, int64_t HW, int64_t C, int groups, int defer_reduce, void* stream);
int64_t pf_groupnorm_workspace(int64_t B, int64_t C, int groups);
/* Number of fp32 workspace elements the column reductions below need. */
int64_t pf_colreduce_workspace(int64_t rows, int64_t cols);
/* acc[c] += sum_r x[r*ld + c]  (bias gradient; deterministic two-stage reduce).
 * Replaces the sum-to-size of aten::addmm's bias gradient + AccumulateGrad. */
int pf_colsum_accumulate(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld, float* acc,
                         float* workspace, int defer_reduce, void* stream);
/* The same reduction for callers that cannot allocate device memory or carry a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the
 * partial rows live in a device array built into the library, pf_colsum_static_capacity()
 * floats (8 MiB) per GPU, held until the process ends.  Always finishes the reduction into
 * `acc` (no deferred mode).  PF_ERR_INVALID when pf_colsum_partials(rows) * cols exceeds the
 * capacity.  Calls that overlap in time on one GPU share the array and race; calls on one
 * stream are ordered.  Allocates nothing.  No counterpart in the reference. */
int pf_colsum_accumulate_static(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld, float* acc,
                                void* stream);
int64_t pf_colsum_static_capacity(void);
/* Deferred column reductions.  With defer_reduce != 0 the three functions above only
 * write their per-workgroup partial rows into `workspace` (layout: norm backward
 * [pf_norm_bwd_partials(rows)][2][d] = dgamma then dbeta partials; column sum
 * [pf_colsum_partials(rows)][cols]) and skip the accumulate; one
 * pf_colreduce_finalize_batch launch then finishes any number of them:
 *   acc[c] += sum_{p < n_partials} ws[p*stride + c]   for c < cols, per item.
 * A backward pass of one stage has ~8 such reductions per transformer block; batching
 * them replaces hundreds of few-microsecond launches by one.  `items_dev` is an array
 * in DEVICE memory.  No counterpart in the reference (it is AccumulateGrad of the bias
 * and normalisation parameters, pfeife/mp/worker.py:1585-1587). */
typedef struct pf_reduce_item {
  const float* ws;
  float* acc;
  int32_t n_partials;
  int32_t reserved;
  int64_t stride;
  int64_t cols;
} pf_reduce_item;
int pf_norm_bwd_partials(int64_t rows);
int pf_colsum_partials(int64_t rows);
int pf_colreduce_finalize_batch(const pf_reduce_item* items_dev, int n_items, int64_t max_cols, void* stream);

/* ---- softmax / attention probabilities ------------------------------------
 * Row softmax over [rows, cols] fp32 scores (row stride ld_s) producing
 * probabilities of dtype p_dtype (row stride ld_p; pad columns cols..ld_p-1 are
 * written as zero so that P can feed pf_gemm with K = cols).  If causal != 0,
 * row r only sees columns c <= (r % q_len) + (cols - q_len).
 * Replaces aten::_softmax inside scaled_dot_product_attention / eager attention. */
int pf_softmax_fwd(const float* s, int64_t ld_s, void* p, int p_dtype, int64_t ld_p, int64_t rows,
                   int64_t cols, int64_t q_len, int causal, void* stream);
/* ds = scale * p * (dp - sum_c(dp*p)); dp fp32 (ld_dp), ds dtype ds_dtype (ld_ds, pad zeroed). */
int pf_softmax_bwd(const float* dp, int64_t ld_dp, const void* p, int p_dtype, int64_t ld_p, void* ds,
                   int ds_dtype, int64_t ld_ds, int64_t rows, int64_t cols, float scale, void* stream);

/* Fused attention: O = softmax(Q K^T * scale [causal]) V and its backward, without the
 * [B,H,Tq,Tk] score matrices in memory.  q/k/v/o and the gradients are [B, H, T, hd]
 * tensors (fp16 or bf16) addressed with ELEMENT strides (batch, head, token) and unit
 * stride along hd, so that heads may sit inside a packed qkv projection.  lse: fp32
 * [B,H,Tq] (written by forward, read by backward); delta: fp32 [B,H,Tq] scratch written
 * and read by backward.  hd must be a multiple of 8 and <= 96 (PF_ERR_UNSUPPORTED
 * otherwise: the caller then uses pf_gemm + pf_softmax).  causal: key j is visible to
 * query i iff j <= i + (Tk - Tq) (bottom-right alignment; for Tq != Tk this is NOT
 * aten::scaled_dot_product_attention's top-left is_causal mask, so the host lowering
 * only passes causal when Tq == Tk).
 * Replaces aten::scaled_dot_product_attention and its backward inside a stage
 * (pfeife/mp/worker.py:1494, :1585-1587). */
typedef struct pf_attn_desc {
  int32_t dtype, B, H, Tq, Tk, hd, causal, reserved;
  float scale;
  float reserved2;
  const void* q; const void* k; const void* v;
  void* o;            /* forward: written; backward: read */
  const void* d_o;
  void* dq; void* dk; void* dv;
  float* lse;
  float* delta;
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, o_st;
  int64_t do_sb, do_sh, do_st, dq_sb, dq_sh, dq_st, dk_sb, dk_sh, dk_st, dv_sb, dv_sh, dv_st;
} pf_attn_desc;
int pf_attention_fwd(const pf_attn_desc* desc, void* stream);
int pf_attention_bwd(const pf_attn_desc* desc, void* stream);

/* ---- losses (pfeife/loss.py:53-70 CrossEntropyLoss / HFCrossEntropyLoss; the
 * mean-reduced nn.CrossEntropyLoss they wrap) -------------------------------
 * logits [rows, classes] (dtype l_dtype, contiguous), targets int64 [rows];
 * rows whose target == ignore_index contribute nothing and are left out of the
 * mean.  row_loss/row_lse: fp32 [rows] scratch kept for backward; loss: fp32 [2]
 * = { mean loss, number of rows that were not ignored }. */
int pf_cross_entropy_fwd(const void* logits, int l_dtype, const int64_t* targets, float* row_loss,
                         float* row_lse, float* loss, int64_t rows, int64_t classes, int64_t ignore_index,
                         void* stream);
/* dlogits = (softmax(logits) - onehot(target)) * (*dloss) / (*n_valid), written
 * as dl_dtype; dloss is a device fp32 scalar (NULL means 1), n_valid is loss+1
 * of the forward call. */
int pf_cross_entropy_bwd(const void* logits, int l_dtype, const int64_t* targets, const float* row_lse,
                         const float* dloss, const float* n_valid, void* dlogits, int dl_dtype, int64_t rows,
                         int64_t classes, int64_t ignore_index, void* stream);
/* Mean squared error (F.mse_loss, bench_models/models/train_sdxl.py:1422-1424):
 * loss[0] = mean((a-b)^2) computed in fp32; partial: fp32 [pf_reduce_workspace(n)]. */
int64_t pf_reduce_workspace(int64_t n);
int pf_mse_fwd(const void* a, int a_dtype, const void* b, int b_dtype, float* partial, float* loss, int64_t n,
               void* stream);
/* da = 2 (a-b) * (*dloss) / n */
int pf_mse_bwd(const void* a, int a_dtype, const void* b, int b_dtype, const float* dloss, void* da,
               int da_dtype, int64_t n, void* stream);
/* loss[0] = sum(x) in fp32 (SumLoss, pfeife/loss.py:9-13). */
int pf_sum_fwd(const void* x, int x_dtype, float* partial, float* loss, int64_t n, void* stream);

/* ---- elementwise (HBM-bound, 16-byte vector accesses) ----------------------
 * Unary activation y = act(x) and its backward dx = dy * act'(x).
 * Replaces aten::gelu / aten::silu / aten::relu and their backward kernels. */
int pf_act_fwd(const void* x, void* y, int dtype, int act, int64_t n, void* stream);
int pf_act_bwd(const void* dy, const void* x, void* dx, int dtype, int act, int64_t n, void* stream);
/* Gated MLP: y = act(gate) * up ; (dgate, dup) from dy.  SwiGLU is act = SILU,
 * GEGLU is act = GELU.  Rows of `cols` elements with independent row strides so
 * that gate/up may be the two halves of one fused projection. */
int pf_glu_fwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* y, int64_t ld_y,
               int dtype, int act, int64_t rows, int64_t cols, void* stream);
int pf_glu_bwd(const void* dy, int64_t ld_dy, const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
               void* dgate, int64_t ld_dgate, void* dup, int64_t ld_dup, int dtype, int act, int64_t rows,
               int64_t cols, void* stream);
/* out = alpha*a + beta*b, each operand with its own dtype (residual add,
 * fan-out gradient sum `g.add_(lg)` of pfeife/mp/worker.py:1543). n elements. */
int pf_axpby(const void* a, int a_dtype, float alpha, const void* b, int b_dtype, float beta, void* out,
             int out_dtype, int64_t n, void* stream);
/* y[r, c] = x[r, c] + bias[row_of_bias(r), c] over n = rows*bias_len elements.
 * rows_per_bias == 0: one bias row broadcast over every row (bias / positional embedding);
 * rows_per_bias  > 0: row r uses bias row r / rows_per_bias (a per-sample vector, e.g. the
 * time-embedding projection added to every pixel of that sample). */
int pf_bias_add(const void* x, int x_dtype, const void* bias, int bias_dtype, void* y, int y_dtype, int64_t n,
                int64_t bias_len, int64_t rows_per_bias, void* stream);
/* dtype conversion / copy of n contiguous elements (autocast's weight casts,
 * done once per optimiser step instead of once per micro-batch). */
int pf_cast(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n, void* stream);
/* Many casts in one launch (`items_dev` in DEVICE memory; vec != 0 promises 16-byte aligned
 * src and dst): the once-per-step refresh of all 16-bit parameter shadows. */
typedef struct pf_cast_item {
  const void* src;
  void* dst;
  int64_t n;
  int32_t src_dtype, dst_dtype, vec, reserved;
} pf_cast_item;
int pf_cast_batch(const pf_cast_item* items_dev, int n_items, int64_t max_n, void* stream);
/* Both 16-bit shadows of many fp32 weight matrices in one launch (`items_dev` in DEVICE memory):
 * plain[r*cols + c] = transposed[c*rows + r] = (dtype) src[r*cols + c]; either destination may
 * be NULL.  Every matrix is contiguous with rows % 4 == 0 and cols % 4 == 0, src 16-byte and
 * the destinations 8-byte aligned (the caller checks; other matrices go through pf_cast_batch /
 * pf_transpose_cast).  max_tiles = max over items of ceil(rows/64) * ceil(cols/64).  The master
 * is read once instead of once per shadow (autocast re-casts the weight at every use). */
typedef struct pf_shadow_item {
  const float* src;
  void* plain;
  void* transposed;
  int64_t rows, cols;
  int32_t dtype, reserved;
} pf_shadow_item;
int pf_shadow_batch(const pf_shadow_item* items_dev, int n_items, int64_t max_tiles, void* stream);
/* dst[c*ld_dst + r] = src[r*ld_src + c] with dtype conversion: the transposed 16-bit
 * shadow of a weight matrix, made once per optimiser step, lets the input-gradient
 * product dx = dy W read W with its reduction dimension contiguous. */
int pf_transpose_cast(const void* src, int src_dtype, int64_t ld_src, void* dst, int dst_dtype, int64_t ld_dst,
                      int64_t rows, int64_t cols, void* stream);
/* dst[i] = value for n elements of a 4-byte or 2-byte float dtype
 * (optimizer.zero_grad(set_to_none=False), pfeife/mp/worker.py:583-597). */
int pf_fill(void* dst, int dtype, float value, int64_t n, void* stream);
/* Generic strided copy with dtype conversion of a tensor of up to 6 dims:
 * dst[idx . dst_strides] = src[idx . src_strides]  (strides in elements). Used
 * for layout changes that are not views: patch extraction, head merges, cat,
 * NCHW <-> NHWC and convolution-weight re-layouts (a copy whose source and destination are
 * contiguous along different dimensions is tiled through LDS as a batched transpose).
 * Integer dtypes (token ids) are copied raw: same dtype on both sides, no accumulate. */
int pf_copy_strided(const void* src, int src_dtype, const int64_t* src_strides, void* dst, int dst_dtype,
                    const int64_t* dst_strides, const int64_t* sizes, int ndim, int accumulate, void* stream);
/* Rotary position embedding (rotate-half convention of HF Llama: element i
 * pairs with i + D/2): x and y are [B, T, H, D] tensors addressed with element
 * strides (sb, st, sh, 1); cos_t/sin_t are fp32 tables with T rows of row
 * stride tab_ld (>= D/2) whose first D/2 columns are used.
 *   y[i]       = x[i] cos[t,i] - x[i+D/2] sin[t,i]
 *   y[i+D/2]   = x[i+D/2] cos[t,i] + x[i] sin[t,i]
 * inverse != 0 applies the transposed rotation (the backward pass). y may alias x. */
int pf_rope(const void* x, void* y, int dtype, const float* cos_t, const float* sin_t, int64_t tab_ld, int64_t B,
            int64_t T, int64_t H, int64_t D, int64_t x_sb, int64_t x_st, int64_t x_sh, int64_t y_sb, int64_t y_st,
            int64_t y_sh, int inverse, void* stream);

/* ---- optimizer step ----------------------------------------------------------------
 * Multi-tensor Adam (adamw = 0: torch.optim.Adam, L2 weight decay added to the gradient;
 * adamw = 1: torch.optim.AdamW, decoupled decay) on fp32 parameters with fp32 gradients
 * and moments, `step` = 1-based step count, one launch per parameter group.  Tensors must be
 * 16-byte aligned; `items_dev` lives in DEVICE memory.  Replaces the foreach kernels of
 * `scaler.step(self.optimizer)` in ProcessWorker.optimizer_step (pfeife/mp/worker.py:1432-1436)
 * for the optimizers `get_optimizer_cls` maps "adam" / "adamw" to (pfeife/option.py:9-29). */
typedef struct pf_adam_item {
  float* param;
  const float* grad;
  float* exp_avg;
  float* exp_avg_sq;
  int64_t n;
} pf_adam_item;
int pf_adam_step(const pf_adam_item* items_dev, int n_items, int64_t max_n, double lr, double beta1, double beta2,
                 double eps, double weight_decay, int64_t step, int adamw, void* stream);

/* ---- dynamic loss scaling on the device ---------------------------------------------
 * torch.amp.GradScaler's rule without a host synchronisation.  `state` is float[8] in DEVICE
 * memory: {scale, growth tracker, found_inf, completed optimizer steps, then four floats of
 * scratch for pf_adam_step_scaled}; the caller initialises it to {init_scale, 0, 0, 0, ...}.
 *   pf_scale_by_state   dst = src * scale          (GradScaler.scale applied to the gradient
 *                                                   entering the last stage)
 *   pf_scaler_unscale   grads *= 1/scale in place; found_inf = 1 if any element is not finite
 *                       (GradScaler.unscale_); call it for every gradient buffer of the step
 *   pf_adam_step_scaled pf_adam_step that does nothing when found_inf is set (GradScaler.step)
 *                       and takes its step count for the bias corrections from the state
 *                       (it writes the two correction terms into state[4..5] first)
 *   pf_scaler_update    GradScaler.update: on overflow scale *= backoff_factor; otherwise the
 *                       step count and the growth tracker advance and every `growth_interval`
 *                       clean steps scale *= growth_factor; clears found_inf
 * Replaces WorkerScaler (pfeife/mp/worker.py:133-145) and scaler.step(optimizer) +
 * scaler.update() (pfeife/mp/worker.py:1432-1436). */
int pf_scale_by_state(const void* src, int src_dtype, const float* state, void* dst, int dst_dtype, int64_t n,
                      void* stream);
int pf_scaler_unscale(float* grads, int64_t n, float* state, void* stream);
int pf_adam_step_scaled(const pf_adam_item* items_dev, int n_items, int64_t max_n, double lr, double beta1,
                        double beta2, double eps, double weight_decay, int adamw, float* scaler_state,
                        void* stream);
int pf_scaler_update(float* state, double growth_factor, double backoff_factor, int growth_interval, void* stream);

/* ---- gradient accumulation --------------------------------------------------
 * acc[i] += g[i] for i < n, acc fp32, g of dtype g_dtype: autograd's
 * AccumulateGrad `param.grad.add_(new_grad)` executed once per parameter per
 * micro-batch by torch.autograd.backward (pfeife/mp/worker.py:1585-1587).
 * Algorithmic traffic: 12 bytes per element for fp32 g. */
int pf_grad_accumulate_f32(float* acc, const void* g, int g_dtype, int64_t n, void* stream);

/* ---- micro-batch split / merge ----------------------------------------------
 * Row gather:  dst[i, :] = src[index ? index[i] : row_start + i, :]  for i < n_rows,
 * rows of row_bytes bytes (any dtype; 16-byte fast path when aligned).
 * With index == NULL this materialises chunk `row_start .. row_start+n_rows` of
 * torch.tensor_split(v, batch_cnt, 0) (pfeife/batch.py:45) as a contiguous slab. */
int pf_split_gather(const void* src, void* dst, int64_t row_bytes, int64_t row_start, int64_t n_rows,
                    const int64_t* index, void* stream);
/* Row scatter: dst[index ? index[i] : row_start + i, :] = src[i, :]; stacks the
 * per-micro-batch results back into one batch-major tensor (the inverse of the
 * split; the reference returns a Python list, pfeife/mp/partial/module.py:99-102). */
int pf_merge_scatter(const void* src, void* dst, int64_t row_bytes, int64_t row_start, int64_t n_rows,
                     const int64_t* index, void* stream);
/* Embedding lookup out[i, :] = table[ids[i], :] with dtype conversion, and its
 * backward dtable[ids[i], :] += dout[i, :] (fp32 accumulate, atomics-free:
 * one wavefront owns a group of table rows and adds in id-list order).  Entries
 * equal to padding_idx (-1: none) contribute nothing, so that row's gradient
 * stays zero.  Replaces aten::embedding(+embedding_dense_backward). */
int pf_embedding_fwd(const void* table, int t_dtype, const int64_t* ids, void* out, int o_dtype, int64_t n_ids,
                     int64_t dim, int64_t vocab, void* stream);
int pf_embedding_bwd(const void* dout, int d_dtype, const int64_t* ids, float* dtable_acc, int64_t n_ids,
                     int64_t dim, int64_t vocab, int64_t padding_idx, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PFEIFE_HIP_H_ */
