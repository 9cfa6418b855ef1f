/*
 * cavs_hip.h -- C ABI of the MI355X (gfx950) backend for Cavs's batched execution
 * of a vertex function F over an instance graph G.
 *
 * This is the boundary the reference's op plug-ins would bind: every entry point
 * replaces the body of one backend::OpImpl::Compute (cavs/backend/op_impl.h:14-28)
 * or one piece of the batching memory manager, and takes what that Compute reads
 * from its OpContext (cavs/midend/op_context.h:14-62) as plain device pointers,
 * row counts, widths and leading dimensions.  No C++ types cross it.
 *
 * Conventions
 *   - every function returns 0 on success or a negative CAVS_E* code and never
 *     aborts (the reference CHECK-aborts, cavs/util/macros_gpu.h:10-45);
 *     cavs_last_error() gives the message of the calling thread's last failure;
 *   - all matrices are row-major fp32; `ld*` is the row stride in elements;
 *   - index lists are device int32 arrays;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     every compute entry point is asynchronous with respect to the device;
 *   - single caller thread per stream, like the reference's session loop.
 */
#ifndef CAVS_HIP_H_
#define CAVS_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  CAVS_OK = 0,
  CAVS_EINVAL = -1,  /* bad argument (shape, alignment, null pointer) */
  CAVS_EHIP = -2,    /* a HIP runtime call failed                      */
  CAVS_ENOMEM = -3,
  CAVS_EUNSUPPORTED = -4
};

const char *cavs_last_error(void);
/* ABI version of this header; bumped on any signature change. */
int cavs_abi_version(void);

/* ------------------------------------------------------------------ runtime
 * Replaces GPUAllocator (cavs/midend/allocator.cu:9-27), the H2D/D2H copies of
 * Tensor feeds (cavs/midend/tensor.cc:324-351), the handle/stream pool
 * (cavs/util/stream_event_handle_pool.h:8-65) and Timing (cavs/util/timing.h:10-67). */
int cavs_init(int device);
int cavs_device_name(char *buf, size_t len);
int cavs_malloc(void **ptr, size_t bytes);
int cavs_free(void *ptr);
int cavs_host_alloc(void **ptr, size_t bytes); /* pinned host memory */
int cavs_host_free(void *ptr);
int cavs_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream);
int cavs_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream);
int cavs_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
/* Tensor::InitWithZero (cavs/midend/tensor.cc:283-300); a fill kernel, safe to
 * capture in a graph. */
int cavs_zero(void *ptr, size_t bytes, void *stream);
int cavs_fill(float *ptr, float value, size_t n, void *stream); /* ConstOp / Fill */
int cavs_stream_create(void **stream);
int cavs_stream_destroy(void *stream);
int cavs_stream_sync(void *stream);
int cavs_event_create(void **event);
int cavs_event_destroy(void *event);
int cavs_event_record(void *event, void *stream);
int cavs_event_sync(void *event); /* host waits until the event has happened */
/* work enqueued on `stream` after this call starts once `event` (recorded on another stream) has happened */
int cavs_stream_wait_event(void *stream, void *event);
int cavs_event_elapsed_ms(float *ms, void *start, void *stop);
/* Kernel timing without brackets of its own on the stream: while the calling thread is armed,
 * the first kernel an entry point launches stamps `start` when it begins executing and every
 * kernel stamps `stop` when it ends, so cavs_event_elapsed_ms(start, stop) is the device time
 * of that entry point's kernels (the interval a kernel trace reports), not launch gaps.
 * cavs_profile_disarm tells whether anything was launched in between.  No counterpart in the
 * reference (it times whole statements on the host, cavs/midend/statement.cc:53-84). */
int cavs_profile_arm(void *start_event, void *stop_event);
int cavs_profile_disarm(int *launched); /* waits for `stop` */

/* A stretch of a stream's work recorded once and enqueued again as one call: everything enqueued on
 * `stream` between cavs_graph_capture_begin and cavs_graph_capture_end is recorded instead of run
 * (kernel launches and copies of this library are fine; nothing in between may wait for the
 * stream or for an event).  cavs_graph_capture_end hands back the replayable graph, or, called with
 * graph_exec = NULL, ends a capture the caller gives up (an error then means the stream did not
 * leave the capture: a capture invalidated by a forbidden call cannot be ended on every runtime).  cavs_graph_launch enqueues the recorded
 * work -- same kernels, same arguments, same order.  For the host loop that re-issues the launches
 * of a batch structure seen before (GraphStatement::Run's round loop, cavs/midend/statement.cc:69-76). */
int cavs_graph_capture_begin(void *stream);
int cavs_graph_capture_end(void *stream, void **graph_exec);
int cavs_graph_launch(void *graph_exec, void *stream);
int cavs_graph_destroy(void *graph_exec);

/* ------------------------------------------------------------------ graph ops
 * Replace GraphGatherOp / GraphScatterOp / GraphPushOp / GraphPullOp /
 * FunctionPopRetOp (cavs/backend/op_impl_graphop.cu:17-327) and their kernels
 * (cavs/backend/functor_batched_memcpy.cuh:18-75).  An id of -1 means "no row":
 * gather writes zeros for it (the reference's separate zero-fill kernel), scatter
 * skips it. */

/* out[b, 0:w] = ids[b] >= 0 ? src[ids[b], 0:w] : 0        b in [0,n) */
int cavs_gather_rows(float *out, int ld_out, const float *src, int ld_src, const int *ids,
                     int n, int w, void *stream);
/* dst[ids[b], 0:w] = inp[b, 0:w]   for ids[b] >= 0 */
int cavs_scatter_rows(float *dst, int ld_dst, const int *ids, const float *inp, int ld_inp,
                      int n, int w, void *stream);
/* out[b, 0:w] = 0 */
int cavs_zero_rows(float *out, int ld_out, int n, int w, void *stream);
/* out[b, 0:w] = inp[b, 0:w]  (Push, Slice, Concat: column blocks via ld) */
int cavs_copy_rows(float *out, int ld_out, const float *inp, int ld_inp, int n, int w,
                   void *stream);
/* out[b, 0:w] += inp[b, 0:w]: PartialAccumulate, the gradient of Slice
 * (BinaryStridedKernel, cavs/backend/op_impl_elementwise.cuh:141-150;
 * cavs/backend/op_impl_elementwise_common.h:97-122) */
int cavs_add_rows(float *out, int ld_out, const float *inp, int ld_inp, int n, int w, void *stream);
/* Both child gathers of a binary vertex function in one pass, plus h_l + h_r:
 *   G[2b+i, 0:w] = ids[2b+i] >= 0 ? pool[ids[2b+i], 0:w] : 0      i in {0,1}
 *   hsum[b, 0:hw] = G[2b, 0:hw] + G[2b+1, 0:hw]   (hsum may be NULL)
 * Replaces the two Gather ops and the Add of apps/paper/tree-lstm-cavs.cc:132-137. */
int cavs_gather_children(float *G, float *hsum, const float *pool, const int *ids, int n,
                         int w, int hw, void *stream);

/* ------------------------------------------------------------------ dense math */
/* Row-major C[M,N] = alpha*op(A)*op(B) + beta*C on the FP32 MFMA pipe.  Replaces
 * MatMulMatCublasWrapper (cavs/backend/cublas_wrapper.cc:12-28) as used by
 * MatMulMatOpCublas (cavs/backend/op_impl_blas3_cublas.cc:34-70) and its
 * gradients (cavs/backend/op_decl_matmul.cc:18-69).  op(A) is M x K. */
int cavs_sgemm(int transA, int transB, int M, int N, int K, float alpha, const float *A,
               int lda, const float *B, int ldb, float beta, float *C, int ldc, void *stream);
/* Bytes of device workspace the two workspace-assisted forms below need for this
 * shape (0 when K is not split). */
size_t cavs_sgemm_splitk_workspace(int M, int N, int K);
/* Same contract as cavs_sgemm for tall-K products with too few output tiles to fill
 * the chip (the deferred weight-gradient GEMMs of
 * cavs/midend/batch_weight_updater.h:12-84): K is split over workgroups, partials go
 * to `workspace` and a second kernel adds them in split order (deterministic).  One
 * call at a time per workspace.  workspace may be NULL (then K is never split). */
int cavs_sgemm_splitk(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                      int lda, const float *B, int ldb, float beta, float *C, int ldc,
                      void *workspace, size_t workspace_bytes, void *stream);
/* cavs_sgemm_splitk without a workspace argument and without any allocation: the K-split
 * partials go to a buffer built into the library's code object (32 MiB per GPU, held until the
 * process ends; cavs_sgemm_splitk_static_max_bytes() returns that size).  No counterpart in the
 * reference: it is for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Same kernels, same plan and
 * bit-for-bit the results of cavs_sgemm_splitk; a shape whose partials would not fit
 * (cavs_sgemm_splitk_workspace(M, N, K) above the maximum) is refused with CAVS_EINVAL -- the
 * number of K splits, and with it the size of the partials, follows the device's CU count, so
 * ask cavs_sgemm_splitk_workspace on the device in question.  A device whose copy of the buffer
 * cannot be found (hipGetSymbolAddress) fails this call only; cavs_init succeeds regardless.  All
 * calls on a GPU share that GPU's buffer: calls that overlap in time on one GPU (two streams,
 * two threads) race; calls on one stream are ordered by it. */
size_t cavs_sgemm_splitk_static_max_bytes(void);
int cavs_sgemm_splitk_static(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                             int lda, const float *B, int ldb, float beta, float *C, int ldc,
                             void *stream);
/* Up to eight independent products C_p = alpha_p*op(A_p)*op(B_p) + beta_p*C_p in one launch
 * (plus one for the K splits): the once-per-step block of
 * cavs/midend/batch_weight_updater.h:12-84 -- the weight-gradient GEMMs -- and the embedding
 * gradient's product next to it.  Each of them alone gives every CU one round of workgroups
 * that load, multiply and store in step; launched together their phases overlap.  Results are
 * those of cavs_sgemm_splitk (fixed summation order).  The outputs must not overlap each other
 * or any input.  cavs_sgemm_group_workspace returns the workspace bytes for the same list. */
typedef struct cavs_gemm_desc {
  int transA, transB, M, N, K;
  float alpha, beta;
  const float *A;
  int lda;
  const float *B;
  int ldb;
  float *C;
  int ldc;
  /* Optional: a block the caller knows about, so that the tiles it covers can stop early.  The
   * rows of a batch that belong to leaves come first in every slab, a leaf gathers zero rows
   * (cavs/backend/op_impl_graphop.cu:77-86) and so its forget gates multiply zero and receive
   * a zero gradient (apps/paper/tree-lstm-cavs.cc:160-171): the f columns of x*W are unused in
   * those rows and the f columns of its gradient are exact zeros there.
   *   CAVS_GEMM_A_ZERO (transA = 0): A[r, k] == 0 for r < zero_rows, k >= zero_col;
   *   CAVS_GEMM_B_ZERO (transB = 0): B[k, c] == 0 for k < zero_rows, c >= zero_col;
   *   CAVS_GEMM_C_UNUSED (beta = 0): C[r, c] is not wanted for r < zero_rows, c >= zero_col and
   *     comes out as the product or as zero.
   * With the zeros where the caller says, results are those without the hint bit for bit (the
   * skipped terms are +-0); a hint is a licence, never an obligation.  0: none. */
  int zero_kind, zero_rows, zero_col;
} cavs_gemm_desc;
enum { CAVS_GEMM_C_UNUSED = 1, CAVS_GEMM_A_ZERO = 2, CAVS_GEMM_B_ZERO = 3 };
size_t cavs_sgemm_group_workspace(int count, const cavs_gemm_desc *products);
int cavs_sgemm_group(int count, const cavs_gemm_desc *products, void *workspace,
                     size_t workspace_bytes, void *stream);
/* cavs_sgemm_group for a caller that enqueues the products on a second stream beside a chain of short
 * dependent launches (the weight gradient of a wide classifier head under the backward rounds,
 * cavs/midend/statement.cc:106-111): the tile launches of products that run alone ask for LDS they do
 * not use, so that at most two of their workgroups share a CU and the chain's workgroups find room
 * on every CU.  Same results. */
int cavs_sgemm_group_beside(int count, const cavs_gemm_desc *products, void *workspace, size_t workspace_bytes,
                            void *stream);
/* cavs_sgemm_group followed by cavs_embed_bwd(dtable, ids, C_k, ldc_k, M_k, N_k) on the result of
 * product k = embed_product (alpha 1, beta 0; its rows are the gradients of looked-up embedding
 * rows): MatMul's input gradient and EmbeddingLookup_grad
 * (cavs/backend/op_impl_blas3_cublas.cc:34-70, op_impl_embedding_lookup.cu:92-148) back to back.
 * The scatter-add runs as extra workgroups of the launch that reduces the other products' K
 * splits and sums product k's own partials itself, so the step has one launch less; C_k still
 * receives the product.  Same workspace as cavs_sgemm_group for the same list. */
int cavs_sgemm_group_embed_bwd(int count, const cavs_gemm_desc *products, int embed_product,
                               float *dtable, const float *ids, void *workspace,
                               size_t workspace_bytes, void *stream);
/* C[r,:] = op(A)*op(B) + D[r >> d_shift, :]: the GEMM and the Accumulate that
 * follows it in the backward of a Mirror'ed operand
 * (cavs/backend/op_decl_slice_join.cc:173-182) in one pass.  Workspace as above. */
int cavs_sgemm_addrows(int transA, int transB, int M, int N, int K, const float *A, int lda,
                       const float *B, int ldb, const float *D, int ldd, int d_shift, float *C,
                       int ldc, void *workspace, size_t workspace_bytes, void *stream);
/* out[j] (+)= sum_r inp[r, j], j in [0,w): UnaryBroadcastingKernel
 * (cavs/backend/op_impl_elementwise.cuh:24-34) used for bias gradients. */
int cavs_colsum(float *out, const float *inp, int ld, int n, int w, int accumulate,
                void *stream);
/* EmbeddingLookupOp / GradOp (cavs/backend/op_impl_embedding_lookup.cu:37-148);
 * ids are floats, the row offset is int(id * E) as in the reference. */
int cavs_embed_fwd(float *out, int ld_out, const float *ids, const float *table, int n, int E,
                   void *stream);
int cavs_embed_bwd(float *dtable, const float *ids, const float *dy, int ld_dy, int n, int E,
                   void *stream);
/* GraphPullOp (cavs/backend/op_impl_graphop.cu:208-258) of the word id and the lookup that
 * follows it (apps/paper/tree-lstm-cavs.cc:139-141) in one pass: ids_out[b] = x[rows[b]],
 * out[b, 0:E] = table[int(ids_out[b] * E) ...]. */
int cavs_embed_pull_fwd(float *out, int ld_out, float *ids_out, const float *x, const int *rows,
                        const float *table, int n, int E, void *stream);
/* cavs_embed_pull_fwd followed by MatMul against B [E, N] (apps/paper/tree-lstm-cavs.cc:139-143:
 * Pull, EmbeddingLookup, MatMul with W) in one launch: C[b, 0:N] = table row of x[rows[b]] times B.
 * The product's A loader reads the table rows through the two lists; the workgroups also leave
 * them in e_out (what the backward pass multiplies by; the column tiles of a row tile share that
 * copying) and the ids in ids_out, exactly as cavs_embed_pull_fwd would.  Results are those of the
 * two calls, bit for bit.  unused_rows, unused_col: C[b, c] with b < unused_rows and
 * c >= unused_col is not wanted (CAVS_GEMM_C_UNUSED above: the f columns of the leaves) and comes
 * out as the product or as zero; 0, 0: everything is wanted. */
int cavs_embed_pull_sgemm(float *C, int ldc, float *e_out, int ld_e, float *ids_out, const float *x,
                          const int *rows, const float *table, int n, int E, const float *B, int ldb,
                          int N, int unused_rows, int unused_col, void *stream);
/* out[r, :] = inp[r, :] + bias[:]  (BinaryBroadcastingKernel,
 * cavs/backend/op_impl_elementwise.cuh:128-139; also the ones-vector bias GEMM of
 * cavs/backend/op_impl_fullyconnected_cublas.cc:74-76) */
int cavs_bias_add_rows(float *out, const float *inp, const float *bias, int n, int w,
                       void *stream);
/* SoftmaxEntropyLossOpCudnn / ...Grad
 * (cavs/backend/op_impl_softmax_entropy_logits_loss.cu:94-140, 212-250):
 * loss[r] = -log softmax(logits[r])[label[r]], dlogits = (softmax - onehot)/n.
 * Either output may be NULL. */
int cavs_softmax_xent(float *loss, float *dlogits, const float *logits, const float *labels,
                      int n, int C, void *stream);
/* The same for n rows out of a batch of n_total (dlogits = (softmax - onehot)/n_total): a loss head
 * that runs chunk by chunk, under the rounds that produce the next chunk's rows.  Row for row the
 * values of the call over the whole batch. */
int cavs_softmax_xent_part(float *loss, float *dlogits, const float *logits, const float *labels,
                           int n, int C, int n_total, void *stream);
/* SGD (cavs/backend/op_impl_sgd.cu): w -= lr * g */
int cavs_sgd(float *w, const float *g, float lr, size_t n, void *stream);

/* ------------------------------------------------------------------ elementwise
 * The un-fused elementwise family (cavs/backend/op_impl_elementwise.{cu,cuh},
 * functor_elementwise.h, op_impl_activation_cudnn.cu).  Operands are read as
 * x[i % count], which covers same-shape, scalar and row-broadcast forms
 * (BinaryKernel / BinaryScalarKernel / BinaryBroadcastingKernel). */
enum {
  CAVS_EW_ADD = 0, CAVS_EW_SUB = 1, CAVS_EW_MUL = 2, CAVS_EW_DIV = 3,
  CAVS_EW_SIGMOID_GRAD = 4, /* a = dy, b = y : dy * y * (1-y)  */
  CAVS_EW_TANH_GRAD = 5,    /* a = dy, b = y : dy * (1 - y*y)  */
  CAVS_EW_RELU_GRAD = 6,    /* a = dy, b = y : y > 0 ? dy : 0  */
  CAVS_EW_EQUAL = 7
};
enum {
  CAVS_EW_ASSIGN = 0, CAVS_EW_NEG = 1, CAVS_EW_ABS = 2, CAVS_EW_SQUARE = 3,
  CAVS_EW_SIGMOID = 4, CAVS_EW_TANH = 5, CAVS_EW_RELU = 6
};
int cavs_ew_binary(int op, float *out, const float *a, size_t na, const float *b, size_t nb,
                   size_t n, int accumulate, void *stream);
int cavs_ew_unary(int op, float *out, const float *a, size_t n, int accumulate, void *stream);
int cavs_scale(float *out, const float *a, float s, size_t n, void *stream); /* Scal */

/* ------------------------------------------------------------------ fused gates
 * The fused-op interface for the three vertex functions the benchmarks use: one
 * kernel replaces the Slice / Add / Sigmoid / Tanh / Mul / Concat chain of F
 * (what the reference's runtime fusion compiler emits as FusedKernel nodes,
 * cavs/midend/runtime_compiler/code_generator.cc:104-185, launched by
 * cavs/backend/op_impl_fused_kernel.cu:34-64) and the chain of F's gradient.
 * Row r of every operand is slab row r of the current round.
 *
 * Tree-LSTM (apps/paper/tree-lstm-cavs.cc:132-171):
 *   xW  [n,4H] (ld_xw) column blocks [i|o|u|f]
 *   hU  [n,3H] blocks [i|o|u], hUf [2n,H] rows (2r: f_l, 2r+1: f_r);
 *        both NULL for a round of leaves (their gathered children are zero)
 *   G   [2n,2H] gathered children, row 2r+i = child i as [h|c]; NULL for leaves
 *   bias [4H] blocks [i|f|u|o]
 *   gates [n,6H] = [i|o|u|f_l|f_r|tanh c] saved for backward; msg [n,2H] = [h|c] */
int cavs_treelstm_gates_fwd(const float *xW, int ld_xw, const float *hU, const float *hUf,
                            const float *G, const float *bias, float *gates, float *msg,
                            int n, int H, void *stream);
/* The same with the Scatter that follows it (cavs/backend/op_impl_graphop.cu:128-190) and Push /
 * FunctionPopRet (:214-318) folded in, for rounds that run their products as separate GEMMs: the
 * message of row r also goes to row pair[r] of the message pool (-1: nowhere) and, if graph_out is
 * given, its h to row out_rows[r] of the graph output.  msg may be NULL then. */
int cavs_treelstm_gates_fwd_scatter(const float *xW, int ld_xw, const float *hU, const float *hUf,
                                    const float *G, const float *bias, float *gates, float *msg,
                                    float *pool, const int *pair, float *graph_out,
                                    const int *out_rows, int n, int H, void *stream);
/* dmsg [n,2H] gathered-back message gradient, dret [n,H] pulled d GraphOutput.
 * Writes dxW [n,4H] (ld_dxw) = [d_i|d_o|d_u|d_fl+d_fr]; for internal rounds also
 * dF [2n,H] = rows (d_fl, d_fr) and the c half of dG [2n,2H] (dc_l, dc_r); pass
 * G = dF = dG = NULL for a round of leaves. */
int cavs_treelstm_gates_bwd(const float *dmsg, const float *dret, const float *gates,
                            const float *G, float *dxW, int ld_dxw, float *dF, float *dG,
                            int n, int H, void *stream);
/* Chain LSTM (apps/paper/seq-lstm-cavs.cc:62-86): a [n,4H] = x*U' (+ h_p*W'),
 * blocks [i|f|u|o]; a2 (optional, may be NULL) is added to a (the h_p*W' term
 * kept in its own buffer); G [n,2H] = [h_p|c_p] or NULL for the first round;
 * gates [n,5H] = [i|f|u|o|tanh c]. */
int cavs_lstm_gates_fwd(const float *a, int ld_a, const float *a2, const float *G,
                        const float *bias, float *gates, float *msg, int n, int H,
                        void *stream);
int cavs_lstm_gates_bwd(const float *dmsg, const float *dret, const float *gates,
                        const float *G, float *da, int ld_da, float *dG, int n, int H,
                        void *stream);
/* Tree-FC (apps/paper/tree-fc-cavs.cc:28-36): h = act(z + bias + x); z, bias, x may
 * each be NULL (z is NULL for a round of leaves).  act: 0 relu, 1 tanh. */
int cavs_treefc_fwd(const float *z, const float *bias, const float *x, float *h, int n, int H,
                    int act, void *stream);
int cavs_treefc_bwd(const float *dh_m, const float *dret, const float *h, float *dz, int n,
                    int H, int act, void *stream);

/* ------------------------------------------------------------------ per-step folds
 * The work of a training step around the rounds, each group in one or two launches.
 *
 * cavs_fc_softmax_xent: FullyConnected (cavs/backend/op_impl_fullyconnected_cublas.cc:71-79)
 * + SoftmaxEntropyLoss (op_impl_softmax_entropy_logits_loss.cu:94-140) and, when dX, dW and db
 * are given, their gradients (:150-163, :212-250) for a head of at most 8 classes:
 * X [n,H], W [C,H], b [C], labels [n] (class ids as floats); loss [n], logits [n,C] (may be
 * NULL), dX [n,H], dW [C,H], db [C]; d logits = (softmax - onehot) / n.  The workspace query
 * returns 0 for a shape this entry point does not take (C > 8, H > 1024, or C * ceil-pow2(H/64) > 64).
 * With dX given and dW, db NULL the weight and bias gradients stay in the workspace as
 * cavs_fc_softmax_xent_parts(n) partial sums of C*H + C floats each, to be added up by a
 * CAVS_TASK_SUM_PARTS job of cavs_run_tasks (n0 = parts, n1 = C*H + C, n2 = C*H). */
size_t cavs_fc_softmax_xent_workspace(int n, int H, int C);
int cavs_fc_softmax_xent_parts(int n);
int cavs_fc_softmax_xent(const float *X, const float *W, const float *b, const float *labels,
                         float *loss, float *logits, float *dX, float *dW, float *db,
                         void *workspace, size_t workspace_bytes, int n, int H, int C, void *stream);
/* SGD (cavs/backend/op_impl_sgd.cu) over `count` tensors in one launch; the arrays are host arrays. */
int cavs_sgd_multi(int count, float *const *w, const float *const *g, const size_t *n, float lr,
                   void *stream);
/* Clip (cavs/backend/op_impl_clip.cu:26-50): scales every gradient in place by
 * clip / max(sum_i ||g_i||_2, clip) -- the sum of the tensors' 2-norms, as the reference adds
 * them; at most 8 non-empty tensors per call; the arrays are host arrays.  After the call
 * workspace[512] holds the factor and workspace[513] the sum of norms (floats). */
size_t cavs_clip_grads_workspace(int count);
int cavs_clip_grads(int count, float *const *g, const size_t *n, float clip, void *workspace,
                    size_t workspace_bytes, void *stream);
/* SGD of an embedding table restricted to the rows ids[0..n) (ids as floats, like
 * EmbeddingLookup).  Equal to the dense update when every other row of dtable is zero.  A row
 * listed several times is updated once: stamp [rows of the table] must start at zero and epoch
 * must grow by one per call. */
int cavs_embed_sgd(float *table, const float *dtable, const float *ids, int n, int E, float lr,
                   int *stamp, int epoch, void *stream);
/* dtable rows ids[0..n) = 0 */
int cavs_embed_zero_rows(float *dtable, const float *ids, int n, int E, void *stream);
/* Column sums of nb (<= 8) adjacent column blocks of bw columns of inp [n, ld], block k written
 * to out block dst_block[k] (a permutation; host array).  Deterministic: row chunks are summed
 * in index order.  The bias gradient of the gates (cavs/backend/op_impl_elementwise.cuh:24-34).
 * With out NULL (dst_block may be NULL too) the chunk sums stay in the workspace as
 * cavs_colsum_parts(n) rows of bw*nb floats, for a CAVS_TASK_BLOCKS_SGD job to add up. */
size_t cavs_colsum_blocks_workspace(int n, int bw, int nb);
int cavs_colsum_parts(int n);
int cavs_colsum_blocks(float *out, const float *inp, int ld, int n, int bw, int nb,
                       const int *dst_block, void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------ fused rounds
 * One round of the Tree-LSTM vertex function (apps/paper/tree-lstm-cavs.cc:129-172)
 * with its graph operators folded in: Gather (op_impl_graphop.cu:50-110) becomes the
 * operand fetch of the recurrent products, Scatter (op_impl_graphop.cu:128-190) the
 * store of the epilogue.  Same operand layouts as the gate kernels above; H must be a
 * multiple of 32.
 *   pool [*,2H] message pool rows [h|c]; child [2n] pool rows of the children of slab
 *   row b at 2b, 2b+1 (-1 = none, reads as zero); pair [n] pool row the message of slab
 *   row b is written to (-1 = nowhere); U = U_iou [H,3H] then U_f [H,H].
 * Writes msg [n,2H] (may be NULL: skipped), pool rows pair[b], and what backward reads again: gates [n,6H],
 * G [2n,2H] (gathered children), hlr [n,H] (h_l + h_r).  With graph_out [*,H] given, the pushed
 * return value h of slab row b is also written to row out_rows[b] (Push + FunctionPopRet,
 * op_impl_graphop.cu:168-206,274-327, folded in). */
int cavs_treelstm_round_fwd(float *pool, const int *child, const int *pair, const float *xW,
                            int ld_xw, const float *U, const float *bias, float *G, float *hlr,
                            float *gates, float *msg, float *graph_out, const int *out_rows, int n,
                            int H, void *stream);
/* cavs_treelstm_round_fwd with the loop's weights read from Upk, the tile-major copy a
 * CAVS_TASK_SGD_PACK job writes (pack(U_iou) [K = H, N = 3H], then pack(U_f) [K = H, N = H] at float
 * 3H*H), which must hold the same values as U.  Same results bit for bit; for the shapes
 * cavs_round_packed_ok(n, H) admits. */
int cavs_treelstm_round_fwd_packed(float *pool, const int *child, const int *pair, const float *xW, int ld_xw,
                                   const float *U, const float *Upk, const float *bias, float *G, float *hlr,
                                   float *gates, float *msg, float *graph_out, const int *out_rows, int n, int H,
                                   void *stream);
/* The same for a round of leaves (no children: gates of x*W + bias only). */
int cavs_treelstm_round_leaves_fwd(float *pool, const int *pair, const float *xW, int ld_xw,
                                   const float *bias, float *gates, float *msg, float *graph_out,
                                   const int *out_rows, int n, int H, void *stream);
/* ------------------------------------------------------------------ the rounds near the roots in one launch
 * The per-round loop of GraphStatement::Run / GraphGradStatement::Run (cavs/midend/statement.cc:
 * 69-76,106-111) for rounds of a few vertices each, as ONE launch per direction.  The caller deals
 * the rows of those rounds to up to 8 groups such that no message passes between groups (whole
 * trees of the batch's message flow per group); a group is run by the H / 16 workgroups of one XCD,
 * which stay resident, keep their share of the recurrent weights in registers and walk the group's
 * rounds behind a barrier of their own (arrival counter and results in that XCD's L2; no L2
 * write-back or invalidate; groups never wait for each other).  Same arithmetic in the same order
 * as cavs_treelstm_round_fwd_packed / cavs_treelstm_round_bwd_children_gates_packed called once
 * per round: results equal bit for bit.
 *   rows (device): the groups' lists of slab rows.  Group g runs nrounds[g] lists one after the
 *   other, list i = rows[start[g * max_rounds + i] .. + count[g * max_rounds + i]), 1..32 rows each
 *   (nrounds, start, count, flags: host arrays).  What a list's rows read must have been written
 *   before the launch or by earlier lists of the same group that it waits for: flags[.] = 2 * w + a,
 *   where the list starts once w of the group's arrivals are in (0: at once -- a further slice of a
 *   round of more than 32 rows) and a = 1 makes the end of the list an arrival (the last slice of a
 *   round).  flags == NULL: every list waits for all the lists before it and arrives.
 *   Every other array is the whole-batch array the per-round entry points take slices of (child
 *   [2N], pair [N], out_rows [N], xW [N,4H], G [2N,2H], hlr [N,H], gates [N,6H], msg [N,2H] or NULL;
 *   backward: dxW [N,4H], dF [2N,H], dc [N,H], child_rows [2N]).
 *   sync: cavs_tail_sync_bytes() of device memory, zero before the first launch; a launch that
 *   completes leaves it zero.  Word 1 is the status: 0, CAVS_TAIL_TIMEOUT (a wait gave up after
 *   spin_max polls: a group's workgroups were not all resident at once) or CAVS_TAIL_SPREAD (they
 *   did not share one XCD).  With a non-zero status every wave has left the kernel, the results of
 *   the launch are undefined, and the caller must clear the block before the next launch.
 *   Launches on one block must not overlap.  extra_arrivals > 0 makes every wait expect that many
 *   more arrivals than there are workgroups: the way to see the give-up path from a test.
 * For H = 512 (cavs_tail_rounds_ok); at most cavs_tail_max_rounds() lists per group. */
enum { CAVS_TAIL_OK = 0, CAVS_TAIL_TIMEOUT = 1, CAVS_TAIL_SPREAD = 2 };
int cavs_tail_rounds_ok(int n, int H);
int cavs_tail_max_rounds(void);
int cavs_tail_max_groups(void);
size_t cavs_tail_sync_bytes(void);
/* Three barriers of the same workgroups with the same footprint and nothing else: tells (through
 * the status word, after the stream has drained) whether this device runs every group's
 * workgroups all at once on one XCD. */
int cavs_tail_probe(unsigned *sync, int H, int spin_max, void *stream);
int cavs_treelstm_tail_fwd(float *pool, const int *child, const int *pair, const float *xW, int ld_xw,
                           const float *Upk, const float *bias, float *G, float *hlr, float *gates,
                           float *msg, float *graph_out, const int *out_rows, const int *rows,
                           int ngroups, const int *nrounds, const int *start, const int *count,
                           const int *flags, int max_rounds, int H, unsigned *sync, int spin_max,
                           int extra_arrivals, void *stream);
int cavs_treelstm_tail_bwd(float *dxW, int ld_dxw, float *dF, float *dc, const float *UTp,
                           const int *child_rows, const float *gates, const float *G,
                           const float *dret, const int *dret_rows, int leaf_rows, const int *rows,
                           int ngroups, const int *nrounds, const int *start, const int *count,
                           const int *flags, int max_rounds, int H, unsigned *sync, int spin_max,
                           int extra_arrivals, void *stream);

/* Backward of the gates of a round.  The message gradient of slab row b is read from
 * dpool row pair[b] (grad of Scatter is Gather on the same list, zero for -1); the c
 * half of the children's message gradients is written to dpool rows child[2b], child[2b+1]
 * (grad of Gather is Scatter).  child, G and dF are all NULL for a round of leaves.  The
 * gradient of the pushed return value of slab row b is dret row b, or row dret_rows[b] when
 * that list is given (grad of FunctionPopRet folded in). */
int cavs_treelstm_round_bwd_gates(float *dpool, const int *pair, const int *child, const float *dret,
                                  const int *dret_rows, const float *gates, const float *G,
                                  float *dxW, int ld_dxw, float *dF, int n, int H, void *stream);
/* The h half: dh_child = [d_i|d_o|d_u] * U_iou^T + d_f(child) * U_f^T written to dpool rows
 * child[2b], child[2b+1].  UT = U_iou^T [3H,H] then U_f^T [H,H] (cavs_transpose). */
int cavs_treelstm_round_bwd_children(const float *dxW, int ld_dxw, const float *dF, const float *UT,
                                     const int *child, float *dpool, int n, int H, void *stream);
/* Both parts of the backward round in one launch, for a batch whose message flow is a forest
 * (every message has exactly one reader): the launch that computes d h of the children of a
 * round (rows [row0, row0 + n) of the whole-batch slabs) goes on to the children's gate
 * gradients and writes the children's rows of dxW / dF and d c of each child to row v of
 * dc [N,H]; the message gradient does not pass through the pool (Scatter_grad followed by the
 * next round's Gather_grad, cavs/backend/op_impl_graphop.cu:137-166 and 45-100, composed).
 * child_rows [2n]: the children of round row b by SLAB row (-1: none); rows below leaf_rows are
 * leaves; dret_rows [N]: the gradient of the return value of slab row v is dret row
 * dret_rows[v].  The rows nobody sends a message to (the roots) get their gate gradients from
 * cavs_treelstm_bwd_gates_rows (message gradient zero) before the first such launch. */
int cavs_treelstm_round_bwd_children_gates(float *dxW, int ld_dxw, float *dF, float *dc, const float *UT,
                                           const int *child_rows, const float *gates, const float *G,
                                           const float *dret, const int *dret_rows, int row0, int n,
                                           int leaf_rows, int H, void *stream);
/* The same launch with the transposed weights in the tile-major layout a CAVS_TASK_PACK_T job
 * writes (UTp = pack(U_iou) [K = 3H, N = H], then pack(U_f) [K = H, N = H] at float 3H*H): a
 * wavefront's weight fragment of a k-group is then one contiguous kilobyte.  For the shapes
 * cavs_round_packed_ok(n, H) admits: rounds of at most 1024 vertices whose kernels split H into
 * whole pipeline stages (H a multiple of 512, or of 128 for rounds above 64 vertices). */
int cavs_round_packed_ok(int n, int H);
int cavs_treelstm_round_bwd_children_gates_packed(float *dxW, int ld_dxw, float *dF, float *dc,
                                                  const float *UTp, const int *child_rows,
                                                  const float *gates, const float *G, const float *dret,
                                                  const int *dret_rows, int row0, int n, int leaf_rows,
                                                  int H, void *stream);
int cavs_treelstm_bwd_gates_rows(const int *rows, int n, const float *dret, const int *dret_rows,
                                 const float *gates, const float *G, float *dxW, int ld_dxw, float *dF,
                                 float *dc, int leaf_rows, int H, void *stream);
/* The same construction for the chain LSTM (apps/paper/seq-lstm-cavs.cc:62-86; one child per
 * vertex: child [n]; Wh [H,4H] blocks [i|f|u|o]; gates [n,5H] = [i|f|u|o|tanh c]; G [n,2H] the
 * gathered predecessor) and for Tree-FC (apps/paper/tree-fc-cavs.cc:28-36; messages are h only:
 * pool [*,H]; W [2H,H]; bias / x may be NULL; G [n,2H] = [h_l|h_r]; act 0 relu, 1 tanh). */
int cavs_lstm_round_fwd(float *pool, const int *child, const int *pair, const float *xW, int ld_xw,
                        const float *Wh, const float *bias, float *G, float *gates, float *msg,
                        float *graph_out, const int *out_rows, int n, int H, void *stream);
int cavs_lstm_round_leaves_fwd(float *pool, const int *pair, const float *xW, int ld_xw,
                               const float *bias, float *gates, float *msg, float *graph_out,
                               const int *out_rows, int n, int H, void *stream);
int cavs_lstm_round_bwd_gates(float *dpool, const int *pair, const int *child, const float *dret,
                              const int *dret_rows, const float *gates, const float *G, float *da,
                              int ld_da, int n, int H, void *stream);
int cavs_treefc_round_fwd(float *pool, const int *child, const int *pair, const float *W,
                          const float *bias, const float *x, float *G, float *msg, float *graph_out,
                          const int *out_rows, int n, int H, int act, void *stream);
int cavs_treefc_round_leaves_fwd(float *pool, const int *pair, const float *bias, const float *x,
                                 float *msg, float *graph_out, const int *out_rows, int n, int H,
                                 int act, void *stream);
/* dz = act'(h) * (d msg read from dpool row pair[b] + d return value) */
int cavs_treefc_round_bwd(const float *dpool, const int *pair, const float *dret, const int *dret_rows,
                          const float *h, float *dz, int n, int H, int act, void *stream);
/* Gradient of the gathered children's h, product and Scatter in one launch: for child p < nchild
 * of slab row b, dpool[child[b*nchild+p]][0:H) = dA[b,0:K) * BT[0:K, p*H:(p+1)*H).  Chain LSTM:
 * nchild 1, dA = da [n,4H], BT = Wh^T [4H,H].  Tree-FC: nchild 2, dA = dz [n,H], BT = W^T [H,2H]. */
int cavs_round_bwd_children(const float *dA, int ld, int K, const float *BT, int ldb, int nchild,
                            const int *child, float *dpool, int pool_width, int n, int H, void *stream);
/* cavs_lstm_round_fwd / cavs_lstm_round_bwd_children_gates with the recurrent weights tile-major:
 * Whp = W' [K = H, N = 4H] as a CAVS_TASK_SGD_PACK job writes it, WhTp = W'^T [K = 4H, N = H] as a
 * CAVS_TASK_PACK_T job does.  Same results bit for bit; for the shapes cavs_lstm_round_packed_ok(n, H)
 * admits (rounds of at most 1024 vertices, H a multiple of 512, or of 256 above 64 vertices). */
int cavs_lstm_round_packed_ok(int n, int H);
int cavs_lstm_round_fwd_packed(float *pool, const int *child, const int *pair, const float *xW, int ld_xw,
                               const float *Whp, const float *bias, float *G, float *gates, float *msg,
                               float *graph_out, const int *out_rows, int n, int H, void *stream);
int cavs_lstm_round_bwd_children_gates_packed(float *da, int ld_da, float *dc, const float *WhTp,
                                              const int *child_rows, const float *gates, const float *G,
                                              const float *dret, const int *dret_rows, int row0, int n,
                                              int leaf_rows, int H, void *stream);
/* The chain LSTM's and Tree-FC's backward round as one launch, as
 * cavs_treelstm_round_bwd_children_gates does it for the Tree-LSTM: whole-batch slabs, the
 * round is rows [row0, row0 + n), child_rows names the children by slab row, and the launch
 * writes the children's rows of da (and d c of each to dc [N,H]) resp. dz.  The rows nobody sends
 * a message to (the last step of every sequence / the roots) come from the *_rows launches. */
int cavs_lstm_round_bwd_children_gates(float *da, int ld_da, float *dc, const float *WhT,
                                       const int *child_rows, const float *gates, const float *G,
                                       const float *dret, const int *dret_rows, int row0, int n,
                                       int leaf_rows, int H, void *stream);
int cavs_lstm_bwd_gates_rows(const int *rows, int n, const float *dret, const int *dret_rows,
                             const float *gates, const float *G, float *da, int ld_da, float *dc,
                             int leaf_rows, int H, void *stream);
int cavs_treefc_round_bwd_children_act(float *dz, const float *WT, const int *child_rows, const float *h,
                                       const float *dret, const int *dret_rows, int row0, int n, int H,
                                       int act, void *stream);
int cavs_treefc_bwd_rows(const int *rows, int n, const float *dret, const int *dret_rows, const float *h,
                         float *dz, int H, int act, void *stream);
/* out [cols,rows] = in [rows,cols]^T */
int cavs_transpose(float *out, const float *in, int rows, int cols, void *stream);
/* Several small jobs that do not depend on each other, in one launch (no counterpart in the
 * reference, where each is an op of its own: cavs/backend/op_impl_sgd.cu,
 * op_impl_embedding_lookup.cu, the transposes cuBLAS does inside its calls).  Results are those
 * of the separate entry points.  At most 12 jobs; a job must not write what another reads.
 *   CAVS_TASK_TRANSPOSE  p0[c][r] = p1[r][c]               n0 rows, n1 columns
 *   CAVS_TASK_ZERO_ROWS  cavs_embed_zero_rows(p0 = dtable, p1 = ids, n0 = n, n1 = E)
 *   CAVS_TASK_SGD        p0[i] -= f0 * p1[i]               i < n0
 *   CAVS_TASK_EMBED_SGD  cavs_embed_sgd(p0 = table, p1 = dtable, p2 = ids, n0 = n, n1 = E,
 *                                       f0 = lr, p3 = stamp, n2 = epoch)
 *   CAVS_TASK_SUM_PARTS  out[i] = sum over p < n0 of p0[p * n1 + i] in a fixed order, i < n1, where
 *                        out[i] is p1[i] for i < n2 and p2[i - n2] above
 *   CAVS_TASK_BLOCKS_SGD p1 holds n1 (<= 8) blocks of n0 floats; block k goes to block d_k of p2 (if
 *                        given) and p0[d_k block] -= f0 * it (if p0 given); d_k = (n2 >> 4k) & 15, a
 *                        permutation.  A gradient that arrives in another block order than its
 *                        parameter's (the gate bias, apps/paper/tree-lstm-cavs.cc:120-123 vs :143-148).
 *                        With P = n2 >> 32 above 1, p1 holds P such rows and the job adds them up first,
 *                        in index order (the chunk sums cavs_colsum_blocks leaves behind).
 *   CAVS_TASK_PACK_T     p0 = B = p1^T (p1 [n0, n1] row-major, so B is [K = n1, N = n0]; n0 a multiple of 16,
 *                        n1 of 64) in the tile-major layout of the packed round entry points: for k-group
 *                        g (16 k) and column tile t (16 columns), floats [((g * N/16 + t) * 256, +256) hold
 *                        B[16g + 4s + c][16t + x] at [s][x][c], s < 4, x < 16, c < 4.
 *   CAVS_TASK_SGD_PACK   p1[i] -= f0 * p2[i] (skipped when p2 is null), then p0 = B = p1 ([K = n0, N = n1]
 *                        row-major; n0 a multiple of 16, n1 of 64) in the same tile-major layout: the
 *                        parameter update (cavs/backend/op_impl_sgd.cu) and the packed copy the next
 *                        forward pass reads, in one pass over the weights.
 *   CAVS_TASK_SGD_TRANSPOSE  p1[i] -= f0 * p2[i] (skipped when p2 is null), then p0[c][r] = p1[r][c], n0 rows,
 *                        n1 columns: the update of a wide classifier's weights [C, H]
 *                        (cavs/backend/op_impl_fullyconnected_cublas.cc:71-79) and the [H, C] copy the
 *                        next step's products read, in one pass.
 *   CAVS_TASK_TREELSTM_GATES_ROWS  cavs_treelstm_bwd_gates_rows(rows = p0, n = n0, dret = p1,
 *                        dret_rows = p2, gates = p3, G = p4, dxW = p5, ld_dxw = n2 >> 32, dF = p6,
 *                        dc = p7, leaf_rows = n2 & 0xffffffff, H = n1; H a multiple of 4): the gate
 *                        gradients of the roots ride in the launch that opens the backward pass.
 *   CAVS_TASK_GUARD      not a job: when the int p0 points at is not zero as the launch runs, none of
 *                        its jobs does anything (the parameter updates of a step whose
 *                        cavs_treelstm_tail_* launch gave up: p0 = the status word of its sync block).
 *                        At most one per launch; it does not count towards the 12.
 * p4 .. p7 are read by CAVS_TASK_TREELSTM_GATES_ROWS only and may stay null otherwise. */
enum { CAVS_TASK_TRANSPOSE = 0, CAVS_TASK_ZERO_ROWS = 1, CAVS_TASK_SGD = 2, CAVS_TASK_EMBED_SGD = 3,
       CAVS_TASK_SUM_PARTS = 4, CAVS_TASK_BLOCKS_SGD = 5, CAVS_TASK_PACK_T = 6, CAVS_TASK_SGD_PACK = 7,
       CAVS_TASK_TREELSTM_GATES_ROWS = 8, CAVS_TASK_SGD_TRANSPOSE = 9, CAVS_TASK_GUARD = 10 };
typedef struct cavs_task {
  int kind;
  float f0;
  long long n0, n1, n2;
  void *p0, *p1, *p2, *p3;
  void *p4, *p5, *p6, *p7;
} cavs_task;
int cavs_run_tasks(int count, const cavs_task *tasks, void *stream);

/* ------------------------------------------------------------------ generic fused op
 * FusedKernelOpImpl (cavs/backend/op_impl_fused_kernel.cu:17-71): compiles the
 * source the fusion pass generated (runtime_compiler/code_generator.cc:20-100;
 * signature: outputs, const inputs, output counts, input counts, n_elements) with
 * the runtime compiler for gfx950, FMA contraction off like the reference's
 * --fmad=false (cavs/backend/cudaRTC_wrapper.h:47-50), and launches it over a 1-D
 * grid. */
int cavs_fused_compile(const char *kernel_name, const char *source, void **handle);
int cavs_fused_launch(void *handle, float *const *outs, int nouts, const float *const *ins,
                      int nins, const int *out_counts, const int *in_counts, int n_elements,
                      void *stream);
int cavs_fused_release(void *handle);
/* The round kernels generated for a vertex function of the general shape, or for one cell of the
 * chain it is cut into (the reference
 * fuses the elementwise operators of F into generated kernels, cavs/midend/runtime_compiler/
 * code_generator.cc:104-185, and runs them through cavs/backend/op_impl_fused_kernel.cu:34-64; here
 * the products of F are inside the generated kernels too).  `source` defines the extern "C" kernels
 * cell_fwd, cell_leaves, cell_bwd, cell_bwd_rows, cell_pack, cell_bias, cell_bwd_gates and
 * cell_bwd_pool, each taking one
 * struct of 8-byte slots by value; cavs_cell_launch passes `args` as that struct.  kernel: index in
 * the order of the names above; block: threads per workgroup (a multiple of 64, at most 256). */
int cavs_cell_compile(const char *source, void **handle);
int cavs_cell_launch(void *handle, int kernel, unsigned grid_x, unsigned grid_y, unsigned grid_z,
                     unsigned block, const void *args, size_t args_bytes, void *stream);
int cavs_cell_release(void *handle);

/* ------------------------------------------------------------------ device schedule
 * The level-wise ready frontier of BatchGraphScheduler::Initialize/ActivateNext
 * (cavs/midend/graph_scheduler.cc:169-245) computed on the GPU from the global
 * parent array.  Inputs: parent[N] (global parent id or -1), N.  Outputs (device,
 * each sized N unless noted): tids_to_jobids, jobids_to_tids, round_of_tid,
 * round2offset [N+2] (entries past R+1 undefined), n_rounds [1]; `scratch` is 4*N
 * ints of device memory the call may overwrite.  Vertices have at most two
 * children, like the reference's two gather lists (graph_scheduler.h:16-18).
 * The backward schedule is these rounds replayed last to first. */
int cavs_schedule_frontier(const int *parent, int N, int *tids_to_jobids, int *jobids_to_tids,
                           int *round_of_tid, int *round2offset, int *n_rounds, int *scratch,
                           void *stream);
/* The whole per-step index arena on the GPU, from the graph feed as the application hands it over
 * (cavs/midend/graph_scheduler.cc:12-71 LoadGraph, :169-245 Initialize / ActivateNext, and the
 * index lists Gather / Scatter / Pull / FunctionPopRet read, cavs/backend/op_impl_graphop.cu:67-76,
 * 148-157,241-249,304-318).  graph: device int32 [B, maxlen], entry j = local parent of vertex j,
 * the first -1 ends the sample; nchild: children of an internal vertex (1 chains, 2 binary trees);
 * pairing: 0 = the reference's (b-th entry of a round's compacted scatter list with slab row b),
 * 1 = row-id preserving.  Outputs, device, `cap` >= B * maxlen rows each:
 *   t2j [cap]            tensor id -> global vertex id (tids_to_jobids)
 *   pair [cap]           slab row -> pool row its message is scattered to / gathered back from, -1 none
 *   child [nchild * cap] slab row, child slot -> pool row of that child (the gather lists), -1 for leaves
 *   kid_rows [nchild * cap]  the same by the slab row that wrote that pool row
 *   roots [B]            vertex ids of the roots;  orphans [B]: slab rows with pair < 0, ascending
 *   meta [maxlen + 9]    [0] N, [1] rounds R, [2] error bits (1 no terminator, 2 parent out of range,
 *                        4 a vertex with children but not `nchild` of them, 8 single-vertex sample,
 *                        16 parent cycle), [3] largest round, [8 + r] round2offset[r] for r <= R.
 * Three dependent launches of one wavefront per sample / one workgroup per round (no grid-wide
 * barrier): the schedule of a batch is the schedules of its samples merged round by round.  With
 * error bits set the lists are undefined.  maxlen <= 2048. */
size_t cavs_schedule_arena_scratch(int B, int maxlen);
int cavs_schedule_arena(const int *graph, int B, int maxlen, int nchild, int pairing, int *t2j, int *pair,
                        int *child, int *kid_rows, int *roots, int *orphans, long cap, int *meta,
                        void *scratch, size_t scratch_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif
