// fp64 building blocks of the CholeskyQR orthonormalisation (see gemm_f64.hip, cholesky.hip).
#pragma once
#include "common.h"

// C[b] (M x N) = alpha * sum_k Aop[b](i,k) Bop[b](j,k) + beta * E[b]   (all of one real type, row-major)
// Operand layouts as in GemmDesc.  E may alias C.  K == 0 is allowed (C = beta * E).
template <typename T>
struct RealGemmDesc {
  const T* A;
  const T* B;
  T* C;
  const T* E;
  long long sA, sB, sC, sE;
  int lda, ldb, ldc, lde;
  int M, N, K, batch;
  int a_kstrided, b_kstrided, symmetric;
  int lower_only;  // 1 (M >= N): only tiles on or below the diagonal (row tile >= column tile) are computed and stored
  double alpha, beta;
  int split_k;   // > 1: K is cut into that many slices (no E term); slice s writes its partial product to
                 // C + s * split_stride and the caller adds the slices in a fixed order (da_auto_split tells it
                 // how many there are).  < 0: the launcher picks the slice count for the tile it chooses
  long long split_stride;   // elements between the outputs of consecutive K slices (>= batch * sC)
  // Optional per-matrix switch: with `gate` set, matrix b is computed only if (gate[b] != 0) == (gate_want != 0);
  // the workgroups of the other matrices return at once.
  const int* gate;
  int gate_want;
  // Storage of C when it is not T (DA_STORE_*): the pointer then addresses elements of that dtype (cast to T*
  // by the caller), ldc and sC count its elements and the result is rounded once at the store.  A converted C
  // excludes E, split_k and the symmetric form.
  int c_store;
  int k_tri;     // 1: B is block lower triangular -- output column tile j only sums k < 64 (j + 1)
};
#define DA_STORE_NATIVE 0
#define DA_STORE_BF16 1
#define DA_STORE_F32 2
inline int da_store_of(int dtype) { return dtype == DA_BF16 ? DA_STORE_BF16 : DA_STORE_F32; }
// Slices of K an auto-split product (split_k < 0) of `blocks` output tiles uses: few tiles with a long K are
// sliced until ~512 workgroups exist.  > 1 means the product leaves that many partial results.
inline int da_auto_split(long long blocks, int K) {
  const int max_split = K / 256 > 0 ? K / 256 : 1;
  const long long sp = (512 + blocks - 1) / blocks;
  return (int)(sp > max_split ? max_split : sp);
}
// Output tiles of the symmetric (Gram) form for `batch` r x r matrices.
inline long long da_gram_blocks(int r, int batch) {
  const long long t = (r + 63) / 64;
  return t * (t + 1) / 2 * batch;
}
typedef RealGemmDesc<double> Gemm64Desc;
typedef RealGemmDesc<float> Gemm32Desc;

// The same kernel in fp32 (v_mfma_f32_16x16x4_f32): the products of the polishing passes, whose input is
// already orthonormal to 1e-4 or better, do not need fp64.
int da_gemm_f32s(const Gemm32Desc& d, hipStream_t s);
int da_gemm_f64(const Gemm64Desc& d, hipStream_t s);

// Conversions of `batch` matrices of `per` contiguous elements each; matrix b is converted only if `gate` is null
// or (gate[b] != 0) == (gate_want != 0).
struct DaGate { const int* flags; int want; };
// dst (f64 / f32) <- src (bf16 / f32)
int da_cvt_to_f64(const void* src, int src_dtype, double* dst, long long per, int batch, DaGate gate, hipStream_t s);
int da_cvt_to_f32(const void* src, int src_dtype, float* dst, long long per, int batch, DaGate gate, hipStream_t s);
// dst (bf16 / f32) <- src (f64)
int da_cvt_from_f64(const double* src, void* dst, int dst_dtype, long long per, int batch, DaGate gate, hipStream_t s);
// dst (f32) <- src (f64 / f32; dst may be null for an f32 source); `low`, if not null, receives the same values in bf16
int da_cvt_f64_to_f32(const double* src, float* dst, bf16_t* low, long long per, int batch, DaGate gate, hipStream_t s);
// h, l (bf16) <- src (f64): h = src rounded to bf16, l = bf16(src - h), i.e. src to 16 bits as h + l
int da_cvt_f64_to_hl(const double* src, bf16_t* h, bf16_t* l, long long per, int batch, DaGate gate, hipStream_t s);
int da_cvt_f32_to_bf16(const float* src, bf16_t* low, long long per, int batch, DaGate gate, hipStream_t s);
// dst (bf16 / f32) <- src (f32)
int da_cvt_from_f32(const float* src, void* dst, int dst_dtype, long long per, int batch, DaGate gate, hipStream_t s);

// Block-column step j = o / 64 of the blocked lower Cholesky G = L L^T of each r x r matrix
// G[b] (o a multiple of 64; nb = 64 except for a ragged last block): factors the nb x nb diagonal
// block at offset o (the trailing updates of earlier steps already applied to G), writes L_jj and
// the panel L[o+nb.., o..o+nb] into Lmat[b], and row block j of W[b] (D_j = L_jj^-1 on the
// diagonal, -D_j L[j, c] left of it).  A non-positive or non-finite pivot zeroes that column (of
// L_jj and of D_j) and records (o + column + 1) in info[b] if it is the matrix's first failure.
// `gate`: as in RealGemmDesc.
// o_prev >= 0 (= o - 64): the trailing update of the previous step, A[i, c] -= L[i, p] L[c, p]^T with p the
// block column at o_prev, has NOT been applied to G; this launch applies it to its own block column before
// use and, with additional workgroups, to the columns o + nb .. c_end - 1 of the lower triangle (in G),
// so that no separate update launch runs between two steps.  Columns >= c_end are left to the caller.
// pstat (fp64 form, may be null): two words per matrix, the smallest and the largest pivot met so far (step o == 0
// starts them): the squares of R's diagonal, whose ratio bounds cond(R)^2 from below.
int da_chol_step(double* G, double* Lmat, double* Wmat, long long sG, int r, int o, int nb, int* info,
                 int batch, DaGate gate, hipStream_t s, int o_prev = -1, int c_end = 0, double* pstat = nullptr);
int da_chol_step_f32(float* G, float* Lmat, float* Wmat, long long sG, int r, int o, int nb, int* info,
                     int batch, DaGate gate, hipStream_t s, int o_prev = -1, int c_end = 0);
// The same step, but instead of the row block of W it writes row block j of T = L^-1 itself into Tmat (lower
// triangular, row-major): T[j, j] = D_j and T[j, c] = -D_j sum_{k = c .. j-1} L[j, k] T[k, c] for c < j, from the
// rows of T that the earlier steps left.  After the last step Tmat holds L^-1 (blocks above the diagonal untouched).
// t_inline = 0: the step leaves the tiles of its row of T left of the diagonal to a later launch (it writes D_j only);
// t_row >= 1: additional workgroups of this launch form those tiles of block row t_row (t_row < j: its D and all rows
// above it are complete), so that the rows of T lag one step behind the factorisation instead of lengthening it.
// da_chol_trow_f32 is that work alone, for the row that is still missing after the last step.
int da_chol_step_f32_inv(float* G, float* Lmat, float* Tmat, long long sG, int r, int o, int nb, int* info,
                         int batch, DaGate gate, hipStream_t s, int o_prev = -1, int c_end = 0, int t_row = -1,
                         int t_inline = 1);
int da_chol_trow_f32(float* Lmat, float* Tmat, long long sG, int r, int t_row, int batch, DaGate gate, hipStream_t s);

#define DA_CHOL_NB 64

// The 16 x 16 x 4 MFMA of either precision: operands are one scalar per lane (A: row = lane % 16,
// k = lane / 16; B: k = lane / 16, column = lane % 16); the four results of a lane are in column
// lane % 16 and rows 4 v + lane / 16 (fp64) resp. 4 (lane / 16) + v (fp32).
template <typename T> struct Mfma;
template <> struct Mfma<double> {
  typedef f64x4_t acc_t;
  static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row(int v, int lane) { return 4 * v + (lane >> 4); }
};
template <> struct Mfma<float> {
  typedef f32x4_t acc_t;
  static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row(int v, int lane) { return 4 * (lane >> 4) + v; }
};

// One 64 x 16 operand tile: 4 elements per thread, fetched into registers (zero filled out of
// range) and later written to lds[k][row].

