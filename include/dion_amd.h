/*
 * dion_amd -- C ABI of the MI355X (gfx950) Muon / Dion optimizer-step kernels.
 *
 * The reference (microsoft/dion) is pure Python on PyTorch and has no FFI of its own:
 * the boundary this library slots in behind is its operator level -- the functions the
 * optimizer classes call on lists of tensors.  Each entry point below names the reference
 * function it replaces (file:line in the reference tree).
 *
 * Conventions
 *   - Plain C types only.  Every pointer is a device pointer unless said otherwise; the
 *     caller owns all memory including the workspace (the library allocates nothing).
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it and nothing
 *     synchronises with the host.
 *   - Matrices are row-major.  dtype codes: DION_AMD_BF16 / _F32 / _F64.
 *   - Return value: 0 ok; <0 argument error (DION_AMD_ERR_*); >0 a hipError_t.
 *   - Alignment: bf16 matrices need every dimension, pitch and batch stride to be a
 *     multiple of 8 elements and 16-byte aligned base pointers (fp32: multiples of 4).
 *     A `workspace` pointer must be 256-byte aligned (the library carves it up itself).
 *     Violations return DION_AMD_ERR_ALIGN; nothing is launched.
 */
#ifndef DION_AMD_H
#define DION_AMD_H
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DION_AMD_BF16 0
#define DION_AMD_F32 1
#define DION_AMD_F64 2

#define DION_AMD_OK 0
#define DION_AMD_ERR_ARG (-1)
#define DION_AMD_ERR_ALIGN (-2)
#define DION_AMD_ERR_WORKSPACE (-3)
#define DION_AMD_ERR_DTYPE (-4)
#define DION_AMD_ERR_LIMIT (-5)

#define DION_AMD_EPI_STORE 0
#define DION_AMD_EPI_AXPBY 1

/* Library version string (static storage). */
const char* dion_amd_version(void);

/* ---------------------------------------------------------------------------------------
 * Newton-Schulz orthogonalisation
 * ------------------------------------------------------------------------------------- */

/* Bytes of workspace dion_amd_newton_schulz wants for `batch` matrices of m x n.  A smaller
 * workspace is accepted as long as one matrix fits: the batch is then processed in chunks. */
size_t dion_amd_ns_workspace_bytes(int batch, int m, int n, int compute_dtype);

/* Replaces zeropower_via_newtonschulz5 (reference dion/muon.py:620-647, twin in
 * dion/newton_schulz_triton.py:305-333 and the Triton driver newton_schulz_triton
 * dion/newton_schulz_triton.py:336-374; fixed-coefficient variant
 * dion/muon_reference.py:10-27).
 *
 * For each of `batch` matrices G_b (m x n, dtype g_dtype, row pitch ldg, batch stride
 * g_stride): cast to compute_dtype, transpose to wide if m > n, divide by
 * (||.||_F + eps), run `steps` iterations  A = X X^T; B = b A + c A A; X = a X + B X  with
 * (a, b, c) = coeffs[3*i .. 3*i+2] (host array), transpose back, store to out_b (m x n,
 * dtype compute_dtype, row pitch ldo, batch stride out_stride).
 * faithful != 0 reproduces every intermediate bf16 rounding of the reference's separate
 * tensor ops inside the GEMM epilogues; 0 rounds once per GEMM. */
int dion_amd_newton_schulz(const void* G, int g_dtype, long long g_stride, int ldg,
                           void* out, long long out_stride, int ldo,
                           int batch, int m, int n,
                           const float* coeffs, int steps, float eps,
                           int compute_dtype, int faithful,
                           void* workspace, size_t workspace_bytes, void* stream);

/* dion_amd_newton_schulz without a workspace argument and without any allocation.  It has no
 * counterpart in the reference: it is for callers that cannot allocate device memory -- code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The working
 * matrices live in an array of DION_AMD_STATIC_SCRATCH_BYTES that is part of the library's
 * device image (every GPU the library runs on holds one copy until the process ends).
 * Same arguments and result as dion_amd_newton_schulz.  One matrix's working set
 * (dion_amd_ns_workspace_bytes(1, m, n, compute_dtype)) must fit the array, else
 * DION_AMD_ERR_LIMIT and nothing is launched; a batch goes through it in chunks.  Every call
 * on a GPU uses that GPU's one array: calls that overlap on one GPU (different streams or
 * threads) race; calls on one stream are ordered and safe. */
#define DION_AMD_STATIC_SCRATCH_BYTES (32u << 20)
size_t dion_amd_static_scratch_bytes(void);
int dion_amd_newton_schulz_static(const void* G, int g_dtype, long long g_stride, int ldg,
                                  void* out, long long out_stride, int ldo,
                                  int batch, int m, int n,
                                  const float* coeffs, int steps, float eps,
                                  int compute_dtype, int faithful, void* stream);

/* Replaces ns_line_1 (reference dion/newton_schulz_triton.py:134-170):
 * C_b (m x m) = A_b A_b^T for A_b (m x k); upper tiles computed, mirrored store. */
int dion_amd_syrk(const void* A, long long a_stride, int lda,
                  void* C, long long c_stride, int ldc,
                  int batch, int m, int k, int dtype, void* stream);

/* Replaces ns_line_2 (reference dion/newton_schulz_triton.py:261-302):
 * C_b = alpha * A_b A_b^T + beta * A_b for symmetric A_b (m x m). */
int dion_amd_sym_poly(const void* A, long long a_stride, int lda,
                      void* C, long long c_stride, int ldc,
                      int batch, int m, float alpha, float beta,
                      int dtype, int faithful, void* stream);

/* General batched GEMM with fused epilogue; replaces the torch matmul / baddbmm / addmm
 * call sites of the hot path (reference dion/newton_schulz_triton.py:363,369;
 * dion/dion.py:801, 839, 1513-1530).
 *   C_b (M x N) = s0 * E_b + s1 * sum_k Aop_b(i,k) Bop_b(j,k)      (epilogue AXPBY)
 *   C_b         = s1 * sum_k ...                                   (epilogue STORE)
 * a_kstrided = 0: A stored M x K (pitch lda); 1: stored K x M.  Same for B (N x K / K x N).
 * in_dtype bf16 or f32; c_dtype (for C and E) bf16 or f32, in any combination.
 * E may alias C. */
int dion_amd_gemm(const void* A, long long a_stride, int lda, int a_kstrided,
                  const void* B, long long b_stride, int ldb, int b_kstrided,
                  void* C, long long c_stride, int ldc,
                  const void* E, long long e_stride, int lde,
                  int batch, int M, int N, int K,
                  int in_dtype, int c_dtype, int epilogue, float s0, float s1,
                  int faithful, void* stream);

/* What the bf16 launcher behind dion_amd_gemm would do with one product of these dimensions
 * (host-side query, nothing is launched; no counterpart in the reference): the tile edge it
 * picks (128 or 256), plus 1 if the product runs the interior-only K loop that stages operands
 * with direct-to-LDS loads.  That loop addresses a tile's operands with 32-bit byte offsets:
 * an operand whose tile spans 4 GiB or more takes the bounds-checked loop instead. */
int dion_amd_gemm_plan(int M, int N, int K, int lda, int a_kstrided, int ldb, int b_kstrided);

/* ---------------------------------------------------------------------------------------
 * Muon step for one bucket of same-shape matrices
 * ------------------------------------------------------------------------------------- */

size_t dion_amd_muon_workspace_bytes(int batch, int m, int n);

/* Replaces muon_update_batch_async on one GPU (reference dion/muon.py:356-391, 437-448,
 * 461-486): muon_update_pre_orthogonalize (525-552), muon_update_newton_schulz (576-593)
 * and muon_update_post_orthogonalize (556-573), batched over a bucket of `batch` matrices
 * of identical shape m x n (create_param_batches, reference dion/opt_utils.py:48-65).
 *
 * X, G, M: HOST arrays of `batch` device pointers (weights, gradients, momentum; contiguous
 * m x n).  x_dtype is the dtype of X and M, g_dtype that of G.  Per matrix, in place:
 *   M <- mu M + G;  U = nesterov ? mu M + G : M;  O = NS(bf16(U));
 *   X <- (1 - lr wd) X - adjusted_lr O.
 * decay = 1 - lr*wd and adjusted_lr are passed as already-evaluated fp32 values. */
int dion_amd_muon_step(void* const* X, const void* const* G, void* const* M,
                       int batch, int m, int n, int x_dtype, int g_dtype,
                       float mu, int nesterov, float decay, float adjusted_lr,
                       const float* coeffs, int steps, float eps, int faithful,
                       void* workspace, size_t workspace_bytes, void* stream);

/* The two element-wise stages of a Muon step on their own, for a caller that supplies its own
 * orthogonalisation (the reference's plug-in hook `newton_schulz_func`, dion/muon.py:48-49,
 * 122-131, called at 585-593).
 *
 * dion_amd_muon_pre replaces muon_update_pre_orthogonalize (reference dion/muon.py:525-552):
 * per matrix  M <- mu M + G (G cast to M's dtype first);  U = bf16(nesterov ? mu M + G : M),
 * with the reference's rounding after every tensor op.  G, M, U: HOST arrays of `batch` device
 * pointers to contiguous m x n matrices (n a multiple of 8); U receives bf16.
 *
 * dion_amd_muon_post replaces muon_update_post_orthogonalize (reference dion/muon.py:556-573):
 * X <- decay X;  X <- X - r_O(adjusted_lr O)  for O of the same shape in o_dtype (bf16 or f32: whatever the
 * orthogonalisation returned; the product adjusted_lr O is rounded to O's dtype as the reference's is). */
int dion_amd_muon_pre(const void* const* G, void* const* M, void* const* U,
                      int batch, int m, int n, int g_dtype, int m_dtype,
                      float mu, int nesterov, void* stream);
int dion_amd_muon_post(void* const* X, const void* const* O,
                       int batch, int m, int n, int x_dtype, int o_dtype,
                       float decay, float adjusted_lr, void* stream);

/* Several buckets (each of one shape) in one call.  Replaces the task generator and the task
 * runtime around muon_update_batch_async (reference dion/muon.py:185-270 _create_muon_tasks,
 * 134-183 step; dion/opt_utils.py AsyncRuntime): where the reference overlaps buckets as
 * concurrent async tasks, here the buckets advance through Newton-Schulz in lock step and
 * each of its three products is ONE grouped launch over up to four buckets, so that a bucket
 * too small to fill the GPU shares it with the others.  Results per matrix are those of
 * dion_amd_muon_step.  Every bucket keeps all its matrices resident in the workspace
 * (no chunking): workspace_bytes must be at least dion_amd_muon_buckets_workspace_bytes(),
 * else DION_AMD_ERR_WORKSPACE and nothing is launched. */
typedef struct dion_amd_muon_bucket {
  void* const* X;        /* HOST arrays of `batch` device pointers, as in dion_amd_muon_step */
  const void* const* G;
  void* const* M;
  int batch, m, n;
  float decay;           /* 1 - lr * weight_decay */
  float adjusted_lr;     /* adjust_lr_* (m, n) applied to lr */
} dion_amd_muon_bucket;

size_t dion_amd_muon_buckets_workspace_bytes(const dion_amd_muon_bucket* buckets, int nbuckets);

int dion_amd_muon_step_buckets(const dion_amd_muon_bucket* buckets, int nbuckets,
                               int x_dtype, int g_dtype, float mu, int nesterov,
                               const float* coeffs, int steps, float eps, int faithful,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Lion / AdamW for the non-matrix parameter groups (embeddings, lm_head, norms, biases)
 * ------------------------------------------------------------------------------------- */

/* Replaces lion_update_foreach (reference dion/scalar_opts.py:152-187; callers
 * dion/muon.py:275-312, dion/dion.py:387-428): one fused in-place pass over `count` tensors.
 * X, G, M: HOST arrays of `count` device pointers (weights, gradients, momentum); numel: HOST
 * array of their lengths (any length; tensors whose pointers are 16-byte aligned move as
 * vectors).  All X share x_dtype, all G g_dtype, all M m_dtype (bf16 or f32).  Per element,
 * with the reference's rounding after every tensor op:
 *   g = G.to(M.dtype); U = sign(lerp(M, g, 1-beta1)); M <- lerp(M, g, 1-beta2);
 *   X <- X * decay; X <- X - U * lr.
 * lr, one_minus_beta1/2 and decay = 1 - lr*weight_decay are passed as already-evaluated fp32
 * values (the reference evaluates them on 0-dim fp32 tensors). */
int dion_amd_lion_step(void* const* X, const void* const* G, void* const* M,
                       const long long* numel, int count,
                       int x_dtype, int g_dtype, int m_dtype,
                       float lr, float one_minus_beta1, float one_minus_beta2, float decay,
                       void* stream);

/* Replaces adamw_update_foreach (reference dion/scalar_opts.py:89-149; callers
 * dion/muon.py:314-353, dion/dion.py:430-473).  V: variance buffers (v_dtype).  Per element:
 *   g = G.to(M.dtype); M <- lerp(M, g, 1-beta1); V <- lerp(V, (g*g).to(V.dtype), 1-beta2);
 *   den = sqrt(V) / bias_correction2_sqrt + epsilon; X <- X * decay;
 *   X <- X - (M / den) * adjusted_lr,
 * with adjusted_lr = lr / (1 - beta1^step) and bias_correction2_sqrt = sqrt(1 - beta2^step)
 * evaluated by the caller in fp32. */
int dion_amd_adamw_step(void* const* X, const void* const* G, void* const* M, void* const* V,
                        const long long* numel, int count,
                        int x_dtype, int g_dtype, int m_dtype, int v_dtype,
                        float adjusted_lr, float one_minus_beta1, float one_minus_beta2, float decay,
                        float bias_correction2_sqrt, float epsilon, void* stream);

/* ---------------------------------------------------------------------------------------
 * Dion step for one bucket of same-shape matrices
 * ------------------------------------------------------------------------------------- */

size_t dion_amd_orthonormalize_workspace_bytes(int batch, int rows, int r);

/* Replaces orthogonalize (reference dion/dion.py:1267-1308; per-matrix variants
 * dion/dion_reference.py:733-789): thin-QR Q factor of each of `batch` contiguous matrices
 * P_b (rows x r, rows >= r, dtype bf16 or f32), written to out_b (same layout; may alias P).
 * Method (passes == 2, the optimizer's case): a blocked CholeskyQR pass (Gram matrix, Cholesky
 * factorisation, triangular solve) in fp32 -- for a bf16 P with its large products on the bf16 matrix
 * cores --, then the Gram matrix of the result, which measures the defect ||P^T P - I||_F the pass left.
 * Where that is at most 2e-3, the first-order form of a second CholeskyQR pass,
 * P <- P (I - up(P^T P - I)), finishes the matrix; the others (and all matrices with rows < 4 r) take the
 * same pass in fp64, flagged and selected on the device: no host synchronisation.
 * passes == 1: the fp64 pass alone; passes == 3: fp64 pass and two polishing passes (each squares the
 * remaining defect).  The factor equals the reference's Householder / randomised Cholesky QR result up to
 * column signs (Cholesky's diagonal is positive).
 * info (device, `batch` ints, may be NULL): 0, or 1 + the first column whose pivot was not positive or
 * whose result was not a unit vector orthogonal to the others (a pivot at round-off level: P is
 * numerically rank deficient) -- the analogue of torch.linalg.cholesky_ex's info; such columns come out as 0. */
int dion_amd_orthonormalize(const void* P, void* out, int dtype, int batch, int rows, int r, int passes,
                            int* info, void* workspace, size_t workspace_bytes, void* stream);

/* The same with the reference's choice of method (`qr_method` of dion/dion_reference.py:733-789, and the
 * fall-back of 752-758), as far as it has a counterpart on the device.  All three yield the thin-QR factor with a
 * positive diagonal of R (the reference's Householder-based variants differ from it by column signs):
 *   DION_AMD_QR_AUTO ("rcqr", what dion_amd_orthonormalize does): a CholeskyQR pass in fp32 first; matrices for
 *     which it fails or leaves ||P^T P - I||_F > 2e-3 go through the fp64 pass; closed-form polishing pass.
 *   DION_AMD_QR_FP64 ("qr"): the fp64 pass and the polishing pass for every matrix.
 *   DION_AMD_QR_CQR  ("cqr"): one CholeskyQR pass in fp32 and nothing else (defect eps32 * cond(P)^2, as in the
 *     reference); a matrix whose factorisation meets a non-positive pivot falls back to the fp64 pass, on the
 *     device, as the reference falls back to the randomised method.  Needs passes == 2. */
#define DION_AMD_QR_AUTO 0
#define DION_AMD_QR_FP64 1
#define DION_AMD_QR_CQR 2
int dion_amd_orthonormalize_method(const void* P, void* out, int dtype, int batch, int rows, int r, int passes,
                                   int qr_method, int* info, void* workspace, size_t workspace_bytes, void* stream);

size_t dion_amd_dion_workspace_bytes(int batch, int m, int n, int r, int m_dtype);
/* 1 if dion_amd_dion_step forms B = M + G inside the launch of P = B Q for a bucket of these dimensions (a chunk of
 * at most 64 matrices at a time), 0 if it runs the addition as a pass of its own (reference dion/dion.py:794, 801).
 * No counterpart in the reference: the benchmark uses it to price that launch's HBM traffic. */
int dion_amd_dion_bq_fused(int batch, int m, int n, int rank, int m_dtype, int g_dtype);

/* Replaces dion_update_ddp with replicate_mesh=None (reference dion/dion.py:742-875) and its
 * helpers tensor_list_to_batch (1200-1218), orthogonalize (1267-1308), fix_all_zero_or_nan
 * (1416-1444), column_normalize (1460-1491), foreach_baddbmm_ (1494-1530) and
 * update_Q_matrix_ (1533-1561), for a bucket of `batch` matrices of identical shape m x n.
 *
 * X, G, M, Q: HOST arrays of `batch` device pointers: weights (m x n, x_dtype), gradients
 * (g_dtype), momentum (m_dtype) and the power-iteration factor Q ((min(m,n)) x r... i.e.
 * n x r when m >= n, m x r when m < n; q_dtype), all contiguous, all updated in place
 * except G.  Per matrix, with B' = B if m >= n else B^T:
 *   B = M + G;  P = orth(B' Q);  R = B'^T P;  (all-zero / NaN guard on P, R)
 *   M <- B - (1-mu) P R^T  (transposed back when m < n);   Q <- R / (||R||_col + eps);
 *   X <- decay X - scaled_lr P Q^T.
 * ef_alpha = -(1 - mu), decay = 1 - lr*wd and scaled_lr = sqrt(m/n)*lr are passed as
 * already-evaluated fp32 values.  Every combination of bf16 / f32 for x, g, m and q is accepted.  info as above.
 * power_iters >= 1 repeats P = orth(B' Q), Q = B'^T P before the updates, the unnormalised R serving as the
 * next Q (reference dion/dion_reference.py:690-730; the batched reference class only allows 1).
 * m and n must be multiples of 8 (the host side pads other shapes with zero rows / columns,
 * which changes no result); the rank r is any value in 1 .. min(m, n): the working matrices
 * carry zero columns up to the next multiple of 8 and Q keeps its r contiguous columns. */
int dion_amd_dion_step(void* const* X, const void* const* G, void* const* M, void* const* Q,
                       int batch, int m, int n, int r,
                       int x_dtype, int g_dtype, int m_dtype, int q_dtype,
                       float ef_alpha, float decay, float scaled_lr, float eps, int faithful,
                       int power_iters,
                       int* info, void* workspace, size_t workspace_bytes, void* stream);

/* dion_amd_dion_step with the orthonormaliser's method chosen by the caller (DION_AMD_QR_*): the per-matrix
 * reference class's `qr_method` (reference dion/dion_reference.py:131-134, 296-299). */
int dion_amd_dion_step_qr(void* const* X, const void* const* G, void* const* M, void* const* Q,
                          int batch, int m, int n, int r,
                          int x_dtype, int g_dtype, int m_dtype, int q_dtype,
                          float ef_alpha, float decay, float scaled_lr, float eps, int faithful,
                          int power_iters, int qr_method,
                          int* info, void* workspace, size_t workspace_bytes, void* stream);

/* The reference's randomised Cholesky QR with the random sketch GIVEN by the caller (the async `orthogonalize`,
 * reference dion/dion.py:1274-1308, whose sketch comes from generate_random_sketch_matrix, 1221-1263; the same
 * sequence in dion/dion_reference.py:764-787):
 *   SP = S P (in P's dtype);  R1 = R-factor of SP;  P1 = P R1^-1;  R2 = chol(P1^T P1);  Q = P1 R2^-1.
 * S: `batch` contiguous sketches of k x rows in P's dtype (k >= r; the reference draws N(0, 1/k) entries with
 * k = 128 ceil(1.25 r / 128)).  R1 is formed as the Cholesky factor of (SP)^T (SP) in fp64 -- the R-factor of a
 * Householder QR of SP up to the signs of its rows -- and the solves and the second factorisation run in fp64 too.
 * rows <= r: the reference factors such a P by Householder QR and draws no sketch (1283-1285); S is then ignored
 * and the fp64 pass of dion_amd_orthonormalize_method runs.  The result is the thin-QR factor with a positive
 * diagonal of R: the reference's up to column signs.  rows, r and k multiples of 8 (bf16) or 4 (f32). */
size_t dion_amd_orthonormalize_sketch_workspace_bytes(int batch, int rows, int r, int k);
int dion_amd_orthonormalize_sketch(const void* P, const void* S, void* out, int dtype, int batch, int rows, int r,
                                   int k, int* info, void* workspace, size_t workspace_bytes, void* stream);

/* dion_amd_dion_step with that orthonormaliser (qr_method "rcqr" of the per-matrix reference class with its own
 * random sketches, reference dion/dion_reference.py:290-294, 764-775).  sketch: power_iters x batch contiguous
 * sketches of sketch_k x max(m, n) in the momentum dtype (device memory), sketch_k a multiple of 8 and >= r. */
size_t dion_amd_dion_sketch_workspace_bytes(int batch, int m, int n, int r, int m_dtype, int sketch_k);
int dion_amd_dion_step_sketch(void* const* X, const void* const* G, void* const* M, void* const* Q,
                              int batch, int m, int n, int r,
                              int x_dtype, int g_dtype, int m_dtype, int q_dtype,
                              float ef_alpha, float decay, float scaled_lr, float eps, int faithful,
                              int power_iters, const void* sketch, int sketch_k,
                              int* info, void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Measurement hooks (no counterpart in the reference; used by the benchmark only)
 * ------------------------------------------------------------------------------------- */

/* When enabled, every kernel launch made by the entry points above is bracketed by a pair
 * of HIP events on its launch stream and tagged with a kernel kind (DION_AMD_PROF_*) and
 * its algorithmic work (flops for GEMM kinds, bytes for the HBM-bound passes). */
#define DION_AMD_PROF_NS_SYRK 0
#define DION_AMD_PROF_NS_POLY 1
#define DION_AMD_PROF_NS_AXPY 2
#define DION_AMD_PROF_STAGE 3
#define DION_AMD_PROF_NORMALIZE 4
#define DION_AMD_PROF_UNSTAGE 5
#define DION_AMD_PROF_GEMM 6
#define DION_AMD_PROF_DION_BQ 7
#define DION_AMD_PROF_DION_BTP 8
#define DION_AMD_PROF_DION_EF 9
#define DION_AMD_PROF_DION_UPD 10
#define DION_AMD_PROF_DION_ORTH 11
#define DION_AMD_PROF_DION_ELEM 12
#define DION_AMD_PROF_SCALAR_OPT 13
#define DION_AMD_PROF_DION_EFUPD 14
#define DION_AMD_PROF_NS_FLOW 15
#define DION_AMD_PROF_KINDS 16
int dion_amd_profile_enable(int on);
int dion_amd_profile_reset(void);
/* Waits for the recorded events of `kind`; returns launch count, summed milliseconds and
 * summed work. */
int dion_amd_profile_read(int kind, long long* launches, double* total_ms, double* total_work);

/* Run-time options of the library (no counterpart in the reference; for tests and measurements that compare two
 * roads through the same entry point within one process).  `name`:
 *   "fused_update"  1: dion_amd_dion_step(_qr) applies error feedback and weight update in one pass over M and X
 *                   where that kernel applies (bf16 momentum, dimensions multiples of 128, rank a multiple of 64);
 *                   0: always as two products with the update in their epilogues (reference dion/dion.py:851-853
 *                   and 865-872 as two calls); -1: the default (one pass unless DION_AMD_NO_FUSED is set in the
 *                   environment).  Both roads give the same bits.
 *   "fused_bq"      Dion's B = M + G: 1 formed inside the launch of P = B Q where that applies (bf16 momentum and
 *                   gradients, the longer dimension a multiple of 256, the shorter of 64); 0 as a pass of its own
 *                   (reference dion/dion.py:794 and 801 as two calls); -1 the default (inside, unless
 *                   DION_AMD_NO_FUSED_BQ is set in the environment).  Both roads give the same bits.
 *   "ns_flow"       how the Newton-Schulz iterations of a bucket set are launched: 0 product by product (three
 *                   grouped launches per iteration); 1 as one persistent launch whenever the shapes allow (wide
 *                   dimensions multiples of 256); 2 the same with an L2 write-back after every tile (cross-check);
 *                   -1 the default: DION_AMD_NS_FLOW in the environment if set, else the persistent launch for
 *                   workloads of many small matrices.  All give the same bits.
 *   "edge_loop"     bf16 products with a ragged dimension on a k-strided operand (Dion's rank-r products at r = 192):
 *                   1 the direct-to-LDS K loop with edge tiles, 0 the bounds-checked K loop, -1 the default (1 unless
 *                   DION_AMD_NO_EDGE_LOOP is set in the environment).  Both give the same bits.
 *   "ns_flow_fail"  test hook: 1 makes every persistent launch start with its status word set, as if a wait had
 *                   run into its limit; the results of such a launch are NaN.
 * The value applies to calls that start after this one returns, on every thread.  Unknown name:
 * DION_AMD_ERR_ARG. */
int dion_amd_set_option(const char* name, int value);

/* Time line of a bf16 GEMM launch (no counterpart in the reference; used by the benchmark only).  While enabled,
 * every workgroup of a bf16 GEMM launch -- one output tile each -- records three readings of the GPU's 100 MHz
 * counter (start, end of its K loop, end of its epilogue) and the hardware id of the CU it ran on.  `read` waits
 * for the device and copies the records of the first `tiles` workgroups (at most 65536) of the most recent such
 * launch to HOST memory: six 64-bit words per tile (t_start, t_k_loop_done, t_end, (XCC id << 32) | HW_ID, and the
 * shader-clock counter at the start and at the end: its difference over that of the 100 MHz counter is the clock the
 * CU ran at). */
int dion_amd_tile_trace_enable(int on);
int dion_amd_tile_trace_read(void* host_dst, int tiles);

/* Ceiling probes (no counterpart in the reference; used by the benchmark only).  which = 0: every wavefront of a
 * launch of one 512-thread workgroup per compute unit issues `iters` x 32 v_mfma_f32_32x32x16_bf16 on operands held in
 * registers, loaded once from `random_src` (device memory, at least compute units x 49152 bytes of random bf16).
 * which = 1: every workgroup streams the same 64 KB of `random_src` (at least compute units / 32 x 65536 bytes) into
 * LDS with direct-to-LDS loads `iters` times.  which = 2: the same 64 KB per pass with 16-byte loads into registers.  which = 3: 16-byte
 * LDS reads only, 64 KB per pass and workgroup.  which = 4: as 0 with v_mfma_f32_16x16x32_bf16 on sixteen accumulators.
 * `records` (device memory, 32 bytes per wavefront = compute units x 256
 * bytes) receives per wavefront the 100 MHz counter and the shader-clock counter at its start and end; `sink`: one
 * float of device memory (never written in practice).  The call waits for the launch and returns its duration
 * between two events on `stream` in *ms. */
int dion_amd_probe(int which, const void* random_src, size_t src_bytes, int iters, void* records, size_t record_bytes,
                   float* sink, double* ms, void* stream);

/* Time line of the persistent Newton-Schulz launch (no counterpart in the reference; used by the benchmark only).
 * While enabled, every tile of such a launch records four readings of the 100 MHz counter -- taken from the queue,
 * dependency met, K loop done, result published -- plus (queue << 48 | (3 * iteration + product) << 32 | ticket) and
 * (XCC id << 32 | HW_ID).  `read` waits for the device and copies up to `max_tiles` records (six 64-bit words each)
 * of the most recent traced launch to HOST memory; *tiles receives their number. */
int dion_amd_ns_flow_trace_enable(int on);
int dion_amd_ns_flow_trace_read(void* host_dst, int max_tiles, int* tiles);

#ifdef __cplusplus
}
#endif
#endif /* DION_AMD_H */
