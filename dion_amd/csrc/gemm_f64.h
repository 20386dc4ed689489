// fp64 building blocks of the CholeskyQR orthonormalisation (see gemm_f64.hip, cholesky.hip).
#pragma once
#include "common.h"

// C[b] (M x N) = alpha * sum_k Aop[b](i,k) Bop[b](j,k) + beta * E[b]   (all fp64, row-major)
// Operand layouts as in GemmDesc.  E may alias C.  K == 0 is allowed (C = beta * E).
struct Gemm64Desc {
  const double* A;
  const double* B;
  double* C;
  const double* E;
  long long sA, sB, sC, sE;
  int lda, ldb, ldc, lde;
  int M, N, K, batch;
  int a_kstrided, b_kstrided, symmetric;
  int lower_only;  // 1 (M == N): only tiles on or below the diagonal are computed and stored
  double alpha, beta;
  int split_k;   // > 1: K is cut into that many slices whose partial products are added atomically into a
                 // zeroed C (no E term); the summation order, and so the last bits, vary run to run
};

int da_gemm_f64(const Gemm64Desc& d, hipStream_t s);
int da_fill_f64(double* p, long long n, double v, hipStream_t s);

// dst (f64) <- src (bf16 / f32), and back; contiguous element counts per call.
int da_cvt_to_f64(const void* src, int src_dtype, double* dst, long long n, hipStream_t s);
int da_cvt_from_f64(const double* src, void* dst, int dst_dtype, long long n, hipStream_t s);

// Block-column step j = o / 64 of the blocked lower Cholesky G = L L^T of each r x r matrix
// G[b] (o a multiple of 64; nb = 64 except for a ragged last block): factors the nb x nb diagonal
// block at offset o (the trailing updates of earlier steps already applied to G), writes L_jj and
// the panel L[o+nb.., o..o+nb] into Lmat[b], and row block j of W[b] (D_j = L_jj^-1 on the
// diagonal, -D_j L[j, c] left of it).  A non-positive or non-finite pivot zeroes that column (of
// L_jj and of D_j) and records (o + column + 1) in info[b] if it is the matrix's first failure.
int da_chol_step(const double* G, double* Lmat, double* Wmat, long long sG, int r, int o, int nb, int* info,
                 int batch, hipStream_t s);

#define DA_CHOL_NB 64
