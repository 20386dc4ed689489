// Diagonal-block step of the batched, blocked fp64 Cholesky used by the CholeskyQR
// orthonormalisation: one workgroup per matrix factors a (<= 64) x (<= 64) block held in
// LDS and inverts the triangular factor, so that the panel solve and the triangular solve
// of P become plain GEMMs (gemm_f64.hip).  No host synchronisation: a failed pivot is
// recorded in a device-side info word, mirroring torch.linalg.cholesky_ex's `info`.
#include "gemm_f64.h"

namespace {

constexpr int NB = DA_CHOL_NB;

// 256 threads as a 16 x 16 grid; thread (bi, bj) keeps the 4 x 4 blocks of the working matrix
// and of the inverse-in-progress at block position (bi, bj) in registers.  Right-looking:
// step c publishes column c of L and row c of L^-1 through LDS, then every thread applies the
// two rank-1 updates to its blocks.  Two barriers per step, no LDS traffic besides the 2 x 64
// published values.
__global__ __launch_bounds__(256) void chol_diag_kernel(const double* __restrict__ G, double* __restrict__ Lmat,
                                                        long long sG, int r, int o, int nb, double* __restrict__ Dinv,
                                                        long long sD, int* __restrict__ info) {
  __shared__ double col[NB];    // column c of L (rows > c), 0 elsewhere
  __shared__ double xrow[NB];   // row c of L^-1
  __shared__ double piv[2];     // sqrt(pivot), 1 / sqrt(pivot)
  __shared__ int first_bad;
  const int b = blockIdx.x, tid = threadIdx.x;
  const int bi = tid >> 4, bj = tid & 15;
  const double* g = G + (long long)b * sG + (long long)o * r + o;
  double a[4][4], y[4][4];
#pragma unroll
  for (int ii = 0; ii < 4; ++ii)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int i = bi * 4 + ii, j = bj * 4 + jj;
      // identity padding beyond nb keeps the padded part inert
      a[ii][jj] = (i < nb && j < nb) ? g[(long long)i * r + j] : (i == j ? 1.0 : 0.0);
      y[ii][jj] = (i == j) ? 1.0 : 0.0;
    }
  if (tid == 0) first_bad = 0;
  __syncthreads();

  for (int cb = 0; cb < NB / 4; ++cb) {
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const int c = cb * 4 + cc;
      if (bi == cb && bj == cb) {
        const double p = a[cc][cc];
        const bool ok = p > 0.0 && p < 1.0e300;  // false for NaN as well
        const double d = ok ? sqrt(p) : 0.0;
        piv[0] = d;
        piv[1] = ok ? 1.0 / d : 0.0;
        if (!ok && c < nb && first_bad == 0) first_bad = o + c + 1;
      }
      __syncthreads();
      const double d = piv[0], di = piv[1];
      if (bj == cb) {  // owners of column c: publish the scaled column, keep L in place
#pragma unroll
        for (int ii = 0; ii < 4; ++ii) {
          const int i = bi * 4 + ii;
          const double l = i > c ? a[ii][cc] * di : 0.0;
          col[i] = l;
          a[ii][cc] = i > c ? l : (i == c ? d : a[ii][cc]);
        }
      }
      if (bi == cb) {  // owners of row c of the inverse-in-progress: X[c, :] = Y[c, :] / L[c][c]
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const double x = y[cc][jj] * di;
          y[cc][jj] = x;
          xrow[bj * 4 + jj] = x;
        }
      }
      __syncthreads();
#pragma unroll
      for (int ii = 0; ii < 4; ++ii) {
        const int i = bi * 4 + ii;
        const double li = col[i];  // 0 for rows <= c
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int j = bj * 4 + jj;
          if (j > c) a[ii][jj] -= li * col[j];
          y[ii][jj] -= li * xrow[j];
        }
      }
    }
  }

  double* l = Lmat + (long long)b * sG + (long long)o * r + o;
  double* di_out = Dinv + (long long)b * sD;
#pragma unroll
  for (int ii = 0; ii < 4; ++ii)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int i = bi * 4 + ii, j = bj * 4 + jj;
      if (i < nb && j < nb) l[(long long)i * r + j] = j <= i ? a[ii][jj] : 0.0;
      di_out[i * NB + j] = (i < nb && j <= i) ? y[ii][jj] : 0.0;
    }
  if (tid == 0 && first_bad != 0 && info[b] == 0) info[b] = first_bad;
}

}  // namespace

int da_chol_diag(const double* G, double* Lmat, long long sG, int r, int o, int nb, double* Dinv, long long sD,
                 int* info, int batch, hipStream_t s) {
  if (nb <= 0 || nb > NB || o < 0 || o + nb > r || batch <= 0) return DA_ERR_ARG;
  hipLaunchKernelGGL(chol_diag_kernel, dim3(batch), dim3(256), 0, s, G, Lmat, sG, r, o, nb, Dinv, sD, info);
  return da_launch_status();
}
