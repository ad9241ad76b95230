/*
 * C ABI of the MI355X (gfx950) implementation of Renee's XFC layer step.
 *
 * Every entry point takes plain device pointers, sizes, leading dimensions (in
 * elements) and an opaque stream (a hipStream_t cast to void*, NULL = default
 * stream).  All work is enqueued on that stream; nothing here synchronises or
 * allocates device memory.  Each returns XFC_OK (0) or one of the XFC_ERR_* codes;
 * nothing ever terminates the process (the reference extension calls exit() on
 * failure: xfc_gemm_kernel.cu:14-22, :102-103, :243-244).
 *
 * Number types: X, W, M (momentum) and G are IEEE half; products accumulate in
 * fp32; dX, dW (when written) and split partial sums are fp32.
 *
 * "reference" below is microsoft/renee; file:line cites its sources.
 */
#ifndef XFC_MI355X_H
#define XFC_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XFC_ABI_VERSION 1

enum {
  XFC_OK = 0,
  XFC_ERR_INVALID = 1,   /* null pointer, negative or > 2^31-1 dimension */
  XFC_ERR_LAYOUT = 2,    /* stride pattern that selects no GEMM mode */
  XFC_ERR_ALIGN = 3,     /* pointer or leading dimension not 16-byte aligned */
  XFC_ERR_WORKSPACE = 4, /* workspace NULL or smaller than *_workspace_bytes() */
  XFC_ERR_HIP = 5,       /* kernel launch failed */
  XFC_ERR_SHAPE = 6,     /* operand shapes disagree / leading dimension too small */
  XFC_ERR_LIMIT = 7      /* problem larger than the fixed capacity of a *_static entry point */
};

const char* xfc_strerror(int code);
int xfc_abi_version(void);

/*
 * Optional set-up for the calling thread's current device: raises the dynamic-LDS limit of
 * every kernel and reads the device's CU count, which the entry points otherwise do on
 * their first launch.  Call it once per device before capturing launches into a graph.
 * No counterpart in the reference (its kernels fit the default shared-memory limit).
 */
int xfc_init(void);

/*
 * The six-argument fused GEMM of the reference extension:
 *   xfc_gemm(mat_in1, mat_in2, mat_out, alpha, beta, apply_sigmoid)   xfc_gemm.cpp:17-40
 * with each 2-D tensor flattened to (pointer, rows, cols, stride0, stride1).
 * M, N come from mat_out and K from mat_in2's rows (xfc_gemm_kernel.cu:49-51);
 * the mode is chosen from the strides of the views passed in, as there:
 *   apply_sigmoid, in1 row-major, in2 column-major:
 *        out(fp16) = sigmoid(alpha*in1.in2 + beta*out)      xfc_gemm_kernel.cu:59-100
 *   in1 column-major, in2 row-major:
 *        out(fp32) = alpha*in1.in2 + beta*out               xfc_gemm_kernel.cu:113-150
 *   in1 row-major, in2 row-major (contraction over the long axis, split):
 *        out(fp32) = alpha*in1.in2 + beta*out               xfc_gemm_kernel.cu:151-241
 * in1 and in2 are fp16.  With beta == 0 the old contents of out are never read.
 * Operands whose leading dimensions are not multiples of 8 elements take a slow
 * any-stride kernel instead of failing.  The row x row mode needs a workspace of
 * xfc_gemm_workspace_bytes(M, N, K) bytes (the reference allocates and frees its
 * split-K workspace inside the call, xfc_gemm_kernel.cu:224-227).
 */
size_t xfc_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int xfc_gemm(const void* in1, int64_t in1_rows, int64_t in1_cols, int64_t in1_s0, int64_t in1_s1,
             const void* in2, int64_t in2_rows, int64_t in2_cols, int64_t in2_s0, int64_t in2_s1,
             void* out, int64_t out_rows, int64_t out_cols, int64_t out_s0, int64_t out_s1,
             float alpha, float beta, int apply_sigmoid,
             void* workspace, size_t workspace_bytes, void* stream);

/*
 * Logits only: out[B x L] (fp16) = X[B x d] . W[L x d]^T.
 * Replaces BCELossMultiNode.xfc_forward, dl_base.py:568-573 (torch.matmul(out=)).
 * ldx, ldw, ldo and d must be multiples of 8 and the pointers 16-byte aligned.
 */
int xfc_logits(const void* X, int64_t ldx, const void* W, int64_t ldw, void* out, int64_t ldo,
               int64_t B, int64_t L, int64_t d, void* stream);

/*
 * Forward + loss gradient in one pass, the loss itself never formed:
 *   G[b][l] = fp16( sigmoid(sum_k X[b][k]*W[l][k]) - [l in positives(b)] )
 * Replaces dl_base.py:591-594 (fused-sigmoid GEMM, then out[pos_x,pos_y] -= 1.0).
 * A (row, label) pair listed more than once lowers G by 1 once, as the
 * reference's non-accumulating indexed update does; pairs outside [0,B)x[0,L)
 * are ignored.  Positives come either as CSR (rowptr int32[B+1], colidx
 * int32[nnz]) or as the reference's COO pair (pos_x, pos_y int64[nnz],
 * dl_base.py:934-936), in any order.  Of colidx the device code reads
 * colidx[max(rowptr[0],0) .. min(rowptr[B],nnz)) and nothing else, each entry
 * once, whatever rowptr holds; row pointers that do not ascend give an
 * unspecified subset of those entries to unspecified rows.
 * G has leading dimension ldg >= L, a multiple of 8; the columns
 * L .. round_up(L,8)-1 are written as zero (xfc_dx / xfc_dw_update rely on it).
 * If `loss` is non-NULL it receives the summed BCE-with-logits loss of the batch,
 *   sum softplus(z) - sum z[positives]          (fp32; Algorithm 1 of the paper,
 * dl_base.py:578-583, which the reference evaluates on one step in 100), from the same
 * pass; positives count once each (the reference's indexed sum would count a duplicated
 * pair twice).  NULL is the --noloss path and costs nothing.
 * Workspace: xfc_fwd_grad_workspace_bytes(L, nnz) bytes.
 */
size_t xfc_fwd_grad_workspace_bytes(int64_t L, int64_t nnz);
int xfc_fwd_grad_csr(const void* X, int64_t ldx, const void* W, int64_t ldw,
                     const int32_t* rowptr, const int32_t* colidx,
                     void* G, int64_t ldg, int64_t B, int64_t L, int64_t d, int64_t nnz,
                     float* loss, void* workspace, size_t workspace_bytes, void* stream);
int xfc_fwd_grad_coo(const void* X, int64_t ldx, const void* W, int64_t ldw,
                     const int64_t* pos_x, const int64_t* pos_y, int64_t nnz,
                     void* G, int64_t ldg, int64_t B, int64_t L, int64_t d,
                     float* loss, void* workspace, size_t workspace_bytes, void* stream);

/*
 * xfc_fwd_grad_csr for callers that cannot allocate device memory or hand over a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results as xfc_fwd_grad_csr minus the workspace: the label buckets
 * live in a fixed XFC_STATIC_SCRATCH_BYTES array inside the library's device image (one copy per GPU,
 * held until the process ends), and the call makes no hipMalloc / hipFree.  Problems whose bucket
 * tables do not fit (xfc_fwd_grad_workspace_bytes(L, nnz) > XFC_STATIC_SCRATCH_BYTES, i.e. beyond
 * about 16.7 M labels with 190 k positives) are rejected with XFC_ERR_LIMIT.  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race;
 * calls in sequence are independent, every table being rebuilt from scratch by each call.
 * Call xfc_init() once per device beforehand (it looks the array's device address up).
 */
#define XFC_STATIC_SCRATCH_BYTES (2 * 1024 * 1024)
int xfc_fwd_grad_csr_static(const void* X, int64_t ldx, const void* W, int64_t ldw,
                            const int32_t* rowptr, const int32_t* colidx,
                            void* G, int64_t ldg, int64_t B, int64_t L, int64_t d, int64_t nnz,
                            float* loss, void* stream);

/*
 * dX[B x d] (fp32) = scale * G[B x L] . W[L x d].
 * Replaces dl_base.py:602-608 (torch.addmm with alpha = loss scale; the dead
 * split-K call at :604).  Needs ldg >= round_up(L,8) with zeroed pad columns
 * (xfc_fwd_grad_* writes them) and a workspace.  xfc_dx_workspace_bytes(B, L, d) is what the
 * fastest split of the label axis needs (slices x B x d x 4 bytes); it is NOT monotone in B (a
 * smaller batch may be cut into more slices), so size a buffer that serves several batch sizes
 * with xfc_layer_workspace_bytes().  A smaller workspace is accepted down to 8 x B x d x 4 bytes:
 * the label axis is then cut into as many slices as fit.
 */
size_t xfc_dx_workspace_bytes(int64_t B, int64_t L, int64_t d);
int xfc_dx(const void* G, int64_t ldg, const void* W, int64_t ldw, float* dX, int64_t lddx,
           int64_t B, int64_t L, int64_t d, float scale,
           void* workspace, size_t workspace_bytes, void* stream);

/*
 * dW = G^T . X, consumed tile by tile by the SGD-momentum update so that W and M
 * make one round trip through memory:
 *   g = dW + weight_decay*W ;  M = momentum*M + g ;  W = W - lr*M
 * (fp32 arithmetic, W and M rounded to fp16 once on store).  Replaces
 * dl_base.py:620-634 (dW GEMM) + dl_base.py:343 (apex FusedSGD.step, parameters
 * main.py:178-179: dampening 0, no Nesterov, decay before momentum).  M must be
 * zero before the first step.  If dW_out is non-NULL the fp32 dW is also written
 * there (leading dimension ld_dw), for checking.
 */
int xfc_dw_update(const void* G, int64_t ldg, const void* X, int64_t ldx,
                  void* W, int64_t ldw, void* M, int64_t ldm,
                  int64_t B, int64_t L, int64_t d,
                  float lr, float momentum, float weight_decay,
                  float* dW_out, int64_t ld_dw, void* stream);

/*
 * The same pass on fp32 master weights and fp32 momentum, i.e. the reference's own optimizer regime
 * (xfc_weight is an fp32 parameter, dl_base.py:185; apex FusedSGD keeps fp32 state, main.py:178-179):
 *   g = dW + weight_decay*W32 ;  M32 = momentum*M32 + g ;  W32 = W32 - lr*M32 ;  W16 = fp16(W32)
 * W16 is the fp16 copy the forward and dX passes read; the reference makes it with a separate cast of
 * the whole matrix every step (dl_base.py:562), here it leaves the update's epilogue.  18 bytes per
 * weight and step against 8 for xfc_dw_update; use it where updates fall below half an fp16 ulp of W
 * (small learning rates, the tail of a cosine schedule), which fp16-resident weights would drop.
 */
int xfc_dw_update_master(const void* G, int64_t ldg, const void* X, int64_t ldx,
                         float* W32, int64_t ldw32, float* M32, int64_t ldm32, void* W16, int64_t ldw16,
                         int64_t B, int64_t L, int64_t d,
                         float lr, float momentum, float weight_decay,
                         float* dW_out, int64_t ld_dw, void* stream);

/*
 * Split gradient accumulation (dl_base.py:318-340, :623-633):
 *   grad[L x d] (fp32) = G^T . X + beta*grad      beta = 0 first micro-batch, 1 after
 * followed once per step by xfc_sgd_momentum over count = L*d contiguous elements.
 */
int xfc_dw(const void* G, int64_t ldg, const void* X, int64_t ldx, float* grad, int64_t ld_grad,
           int64_t B, int64_t L, int64_t d, float beta, void* stream);
int xfc_sgd_momentum(void* W, void* M, const float* grad, int64_t count,
                     float lr, float momentum, float weight_decay, void* stream);
/* ... and its fp32-master form (W32, M32 updated, W16 = fp16(W32) written), see xfc_dw_update_master. */
int xfc_sgd_momentum_master(float* W32, float* M32, void* W16, const float* grad, int64_t count,
                            float lr, float momentum, float weight_decay, void* stream);

/*
 * One whole step for one batch (dl_base.py:303-344 with accum == 1):
 * xfc_fwd_grad_csr, xfc_dx (with W before the update), xfc_dw_update.
 * G is caller-provided scratch of B x ldg halves, ldg >= round_up(L,8)
 * (the reference's preallocated `outsoft`, dl_base.py:176).
 */
size_t xfc_step_workspace_bytes(int64_t B, int64_t L, int64_t d, int64_t nnz);
int xfc_step_csr(const void* X, int64_t ldx, void* W, int64_t ldw, void* M, int64_t ldm,
                 const int32_t* rowptr, const int32_t* colidx, int64_t nnz,
                 void* G, int64_t ldg, float* dX, int64_t lddx,
                 int64_t B, int64_t L, int64_t d,
                 float lr, float momentum, float weight_decay, float scale,
                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * Exact top-K labels per query row over all L labels:
 *   values[b][0..K-1], indices[b][0..K-1] = the K largest X[b].W[l], ties broken towards
 *   the lower label id.
 * Replaces FullPredictor's scoring loop, dl_base.py:736-756 (xfc_forward into outsoft,
 * then torch.max K times with the winners overwritten, or torch.topk for K > 5) and the
 * pad clamp at dl_base.py:782: indices >= numy are returned as numy-1.  1 <= K <= 8192, K <= L.
 *   K <= 8 (the reference's per-epoch K = 5): one fused pass, the logits are never
 *     written; values are the fp32 accumulators (the reference returns fp16-rounded logits).
 *   8 < K <= 8192 (the reference's final evaluation, K = 100, dl_base.py:817-818; torch.topk at
 *     dl_base.py:756 takes any K; above 1024 the selection sorts in a 128 KB LDS buffer, one row per CU): the fp16
 *     logits of a block of rows go to the workspace and an exact selection kernel picks each
 *     row's K largest; values are those fp16 logits widened to fp32, ties are between equal
 *     fp16 values.  xfc_topk_workspace_bytes() asks for all B rows at once (B*round_up(L,8)*2
 *     bytes); any 16-byte aligned workspace that holds min(B, 256) rows is accepted and the
 *     rows are then processed in blocks of a multiple of 256.
 * Scores are expected to be finite: NaN and -inf are never selected by the K <= 8 pass, and a row with
 * fewer than K selectable scores reports (-inf, numy-1) in the remaining places.
 * Workspace: 16-byte aligned (for every K), xfc_topk_workspace_bytes(B, L, K) bytes.  For K <= 8 that is
 * the need of the fastest plan (label groups x B x K x 8 bytes and small extras) and is NOT monotone in B (a
 * smaller batch has fewer row tiles and so more label groups); a smaller workspace is accepted down to the
 * need of 8 label groups.  Use xfc_layer_workspace_bytes() for a buffer that serves every batch size.
 */
size_t xfc_topk_workspace_bytes(int64_t B, int64_t L, int64_t K);
int xfc_topk(const void* X, int64_t ldx, const void* W, int64_t ldw,
             int64_t B, int64_t L, int64_t d, int64_t numy, int K,
             float* values, int64_t* indices,
             void* workspace, size_t workspace_bytes, void* stream);

/*
 * One workspace for every call of a layer: the largest need of xfc_step_csr (= xfc_fwd_grad_* + xfc_dx)
 * and of xfc_topk with K <= 8 over all batch sizes 1..max_batch, with at most max_nnz label pairs per
 * batch.  The per-call *_workspace_bytes() functions are not monotone in B, so sizing by max_batch alone
 * does not cover the smaller batches (the last partial batch of an epoch, --accum micro-batches:
 * dl_base.py:318-340 runs any batch up to xfc_batch_size on the buffers allocated at dl_base.py:175-187).
 */
size_t xfc_layer_workspace_bytes(int64_t max_batch, int64_t L, int64_t d, int64_t max_nnz);

/*
 * Plain device-to-device copy of `bytes` bytes (a multiple of 16, 16-byte aligned
 * pointers).  No counterpart in the reference: it is the kernel of known size against
 * which the HBM traffic counters (FETCH_SIZE / WRITE_SIZE) of the other kernels are
 * scaled when profiling, and a convenient way to snapshot W or M on a stream.
 */
int xfc_copy(const void* src, void* dst, int64_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* XFC_MI355X_H */
