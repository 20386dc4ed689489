// Diagonal-block step of the batched, blocked fp64 Cholesky used by the CholeskyQR
// orthonormalisation: one workgroup per matrix factors a (<= 64) x (<= 64) block held in
// LDS and inverts the triangular factor, so that the panel solve and the triangular solve
// of P become plain GEMMs (gemm_f64.hip).  No host synchronisation: a failed pivot is
// recorded in a device-side info word, mirroring torch.linalg.cholesky_ex's `info`.
#include "gemm_f64.h"

namespace {

constexpr int NB = DA_CHOL_NB;

// 256 threads as a 16 x 16 grid; thread (bi, bj) keeps the 4 x 4 blocks of the working matrix
// and of the inverse-in-progress at block position (bi, bj) in registers.  Right-looking with
// 4-wide block columns: per block step the diagonal owner factors and inverts its 4 x 4 block
// in registers, the column owners form their L blocks (A_ic * L_cc^-T), the row owners of the
// inverse form X_c = L_cc^-1 * Y_c, both are published through LDS, and every thread applies
// the two rank-4 updates.  Two barriers per 4 columns.
__global__ __launch_bounds__(256) void chol_diag_kernel(const double* __restrict__ G, double* __restrict__ Lmat,
                                                        long long sG, int r, int o, int nb, double* __restrict__ Dinv,
                                                        long long sD, int* __restrict__ info) {
  __shared__ double dinv4[4][4];       // inverse of the current diagonal 4 x 4 factor (lower)
  __shared__ double dfac4[4][4];       // the factor itself
  __shared__ double lcol[NB][4];       // rows > 4cb+3: L[i][4cb .. 4cb+3]
  __shared__ double xrow[4][NB];       // rows 4cb .. 4cb+3 of L^-1
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
    if (bi == cb && bj == cb) {
      // unblocked Cholesky of the 4 x 4 diagonal block and its inverse, in registers
      double di[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const double p = a[c][c];
        const bool ok = p > 0.0 && p < 1.0e300;  // false for NaN as well
        const double d = ok ? sqrt(p) : 0.0;
        di[c] = ok ? 1.0 / d : 0.0;
        if (!ok && cb * 4 + c < nb && first_bad == 0) first_bad = o + cb * 4 + c + 1;
        a[c][c] = d;
#pragma unroll
        for (int i = c + 1; i < 4; ++i) a[i][c] *= di[c];
#pragma unroll
        for (int i = c + 1; i < 4; ++i)
#pragma unroll
          for (int j = c + 1; j <= i; ++j) a[i][j] -= a[i][c] * a[j][c];
      }
      double inv[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          double t = (i == j) ? 1.0 : 0.0;
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (k >= j && k < i) t -= a[i][k] * inv[k][j];
          inv[i][j] = j <= i ? t * di[i] : 0.0;
        }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (j > i) a[i][j] = 0.0;
          dfac4[i][j] = a[i][j];
          dinv4[i][j] = inv[i][j];
        }
    }
    __syncthreads();
    if (bj == cb && bi > cb) {
      // L_ic = A_ic * L_cc^-T : row ii of the block times the transposed inverse
      double l[4][4];
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          double t = 0.0;
#pragma unroll
          for (int k = 0; k < 4; ++k) t += a[ii][k] * dinv4[jj][k];
          l[ii][jj] = t;
        }
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          a[ii][jj] = l[ii][jj];
          lcol[bi * 4 + ii][jj] = l[ii][jj];
        }
    }
    if (bi == cb) {
      // X_c = L_cc^-1 * Y_c  (rows 4cb .. 4cb+3 of the inverse are final after this)
      double x[4][4];
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          double t = 0.0;
#pragma unroll
          for (int k = 0; k < 4; ++k) t += dinv4[ii][k] * y[k][jj];
          x[ii][jj] = t;
        }
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          y[ii][jj] = x[ii][jj];
          xrow[ii][bj * 4 + jj] = x[ii][jj];
        }
    }
    __syncthreads();
    if (bi > cb) {
      double li[4][4];
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int k = 0; k < 4; ++k) li[ii][k] = lcol[bi * 4 + ii][k];
      if (bj > cb) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const double lj = lcol[bj * 4 + jj][k];
#pragma unroll
            for (int ii = 0; ii < 4; ++ii) a[ii][jj] -= li[ii][k] * lj;
          }
      }
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const double xk = xrow[k][bj * 4 + jj];
#pragma unroll
          for (int ii = 0; ii < 4; ++ii) y[ii][jj] -= li[ii][k] * xk;
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
