// Host-side interfaces of the Dion building blocks (dion.hip).
#pragma once
#include "common.h"
#include "elementwise.h"

int da_fill_int(int* p, int n, int v, hipStream_t s);
// dst_a[i] = ta.p[i], dst_b[i] = tb.p[i], nonzero[i] = info[i] = 0 for i < n <= DA_MAX_PTRS, in one launch.
int da_dion_setup(const DaPtrTable& ta, void** dst_a, const DaPtrTable& tb, void** dst_b, int n, int* nonzero,
                  int* info, hipStream_t s);
int da_add_grad(const DaPtrTable& m, const DaPtrTable& g, int m_dtype, int g_dtype, long long n, int batch,
                int* nonzero, hipStream_t s);
// dst[b] (rows x ld, contiguous batch) <- table[b] (rows x cols contiguous), columns beyond cols zeroed; ld % 8 == 0.
int da_cast_table(const DaPtrTable& src, int s_dtype, void* dst, int d_dtype, int rows, int cols, int ld, int batch,
                  hipStream_t s);
int da_fix(void* v, const void* alt, int dtype, long long n, int batch, const int* nonzero, hipStream_t s);
// v[b] <- fix(round(part[0][b] + ... + part[parts-1][b])): the partial sums (fp32, n elements per matrix, slice k
// at part + k * pstride) of a product whose inner dimension was cut into slices.
int da_fix_sum(const float* part, int parts, long long pstride, void* v, const void* alt, int dtype, long long n,
               int batch, const int* nonzero, hipStream_t s);
// R, qn: rows x r (r % 8 == 0); the Q state receives the first q_cols columns as a contiguous rows x q_cols
// matrix.  `sums` is scratch for (1 + min(ceil(rows / 64), 1024)) * batch * r doubles.
int da_colnorm(const void* R, void* qn, int m_dtype, const DaPtrTable& q, int q_dtype, int rows, int r, int q_cols,
               float eps, int batch, double* sums, hipStream_t s);

// CholeskyQR (passes = 1) / CholeskyQR2 (passes = 2) of `batch` contiguous matrices P[b]
// (rows x r, dtype bf16 or f32): one pass with fp64 Gram, Cholesky and triangular solve, then
// passes - 1 first-order polishing passes in fp32; result in `out` (same dtype and layout, may
// alias P).  info[b] receives 1 + the first failed pivot
// column (0 = success); failed columns come out as zeros.  Columns r_live .. r-1 of P are zero
// padding (r_live == r: none) and stay zero.
size_t da_orth_workspace_bytes(int batch, int rows, int r);
// method: how the first pass is chosen (the reference's qr_method, dion/dion_reference.py:733-789)
#define DA_QR_AUTO 0   // "rcqr": CholeskyQR in fp32, its measured defect sends a matrix on to the fp64 pass
#define DA_QR_FP64 1   // "qr": the fp64 pass for every matrix
#define DA_QR_CQR 2    // "cqr": one CholeskyQR pass in fp32 and nothing else; a failed factorisation falls back to DA_QR_AUTO's fp64 pass
int da_orthonormalize(const void* P, void* out, int dtype, int batch, int rows, int r, int r_live, int passes,
                      int method, void* ws, int* info, hipStream_t s);

// Randomised Cholesky QR with a sketch given by the caller (reference dion/dion.py:1287-1303): S is batch x k x rows
// in P's dtype (k >= r_live); `extra`: da_orth_sketch_extra_bytes(batch, k, r) bytes beyond `ws`.
size_t da_orth_sketch_extra_bytes(int batch, int k, int r);
int da_orthonormalize_sketch(const void* P, const void* S, void* out, int dtype, int batch, int rows, int r, int r_live,
                             int k, void* ws, void* extra, int* info, hipStream_t s);

// B = M + G and P = B Q in one launch (dion_bq.hip; reference dion/dion.py:794, 801): the product's row operand is
// formed from M and G on the way into LDS and written back over M.  tabM / tabG: the matrices (bf16, row pitch ldm;
// `transposed`: B is the transpose of what is stored, mp x np either way); Q: batch x np x ldq, P: batch x mp x ldq
// (bf16, r live columns); nonzero[b] is set when some element of B[b] is not zero.  Computes the first 256 columns of
// P; the caller launches the plain product for the others (on the B this launch leaves in M).  Same bits as the two
// launches.
bool da_dion_bq_sum_applicable(int batch, int mp, int np, int r, int ldm, int transposed, int m_dtype, int g_dtype);
int da_dion_bq_sum(const DaPtrTable& tabM, const DaPtrTable& tabG, const void* Q, void* P, long long sQ, long long sP,
                   int* nonzero, int batch, int mp, int np, int r, int ldq, int ldm, int transposed, int faithful,
                   hipStream_t s);

// Error feedback and weight update in one pass (dion_fused.hip), bf16 factors:
//   M[b] <- M[b] + ef_alpha P[b] R[b]^T,  X[b] <- decay X[b] - scaled_lr P[b] Qn[b]^T   (R P^T, Qn P^T when `transposed`)
// with every rounding of the reference's separate tensor ops.  P: batch x mp x r, R / Qn: batch x np x r (contiguous);
// tabM / tabX: the matrices (row pitch ldo; momentum bf16, weights x_dtype), at most DA_MAX_PTRS of them.
// Applicable when mp and np are multiples of 128 and r of 64.
bool da_dion_ef_update_applicable(int mp, int np, int r, int m_dtype);
int da_dion_ef_update(const void* P, const void* R, const void* Qn, const DaPtrTable& tabM, const DaPtrTable& tabX, int batch,
                      int mp, int np, int r, int ldo, int transposed, int x_dtype, float ef_alpha, float decay,
                      float scaled_lr, hipStream_t s);
