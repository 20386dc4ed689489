// Diagonal-block step of the batched, blocked fp64 Cholesky used by the CholeskyQR
// orthonormalisation: one workgroup per matrix factors a (<= 64) x (<= 64) block held in
// LDS and inverts the triangular factor, so that the panel solve and the triangular solve
// of P become plain GEMMs (gemm_f64.hip).  No host synchronisation: a failed pivot is
// recorded in a device-side info word, mirroring torch.linalg.cholesky_ex's `info`.
#include "gemm_f64.h"

namespace {

constexpr int NB = DA_CHOL_NB;
constexpr int LP = NB + 1;  // LDS pitch

__global__ __launch_bounds__(256) void chol_diag_kernel(const double* __restrict__ G, double* __restrict__ Lmat,
                                                        long long sG, int r, int o, int nb, double* __restrict__ Dinv,
                                                        long long sD, int* __restrict__ info) {
  __shared__ double a[NB * LP];     // working block, becomes L (lower)
  __shared__ double inv[NB * LP];   // L^-1 (lower)
  __shared__ double dinv[NB];       // 1 / L[c][c], 0 for a failed pivot
  __shared__ int first_bad;
  const int b = blockIdx.x, tid = threadIdx.x;
  const double* g = G + (long long)b * sG + (long long)o * r + o;
  if (tid == 0) first_bad = 0;
  for (int e = tid; e < NB * NB; e += 256) {
    const int i = e / NB, j = e % NB;
    a[i * LP + j] = (i < nb && j < nb) ? g[(long long)i * r + j] : 0.0;
    inv[i * LP + j] = 0.0;
  }
  __syncthreads();

  for (int c = 0; c < nb; ++c) {
    // every thread reads the (fully updated) column c and its pivot
    const double p = a[c * LP + c];
    const bool ok = p > 0.0 && p < 1.0e300;  // false for NaN as well
    const double d = ok ? sqrt(p) : 0.0;
    const double di = ok ? 1.0 / d : 0.0;
    // trailing update of the lower triangle right of column c with the scaled column
    for (int e = tid; e < NB * NB; e += 256) {
      const int i = e / NB, j = e % NB;
      if (i > c && j > c && j <= i && i < nb) a[i * LP + j] -= (a[i * LP + c] * di) * (a[j * LP + c] * di);
    }
    __syncthreads();
    // now scale column c in place (nobody reads it unscaled any more)
    if (tid < nb && tid > c) a[tid * LP + c] *= di;
    if (tid == 0) {
      a[c * LP + c] = d;
      dinv[c] = di;
      if (!ok && first_bad == 0) first_bad = o + c + 1;
    }
    __syncthreads();
  }

  // inverse of the lower-triangular factor: thread c solves L x = e_c by forward substitution
  if (tid < nb) {
    const int c = tid;
    for (int i = c; i < nb; ++i) {
      double s = (i == c) ? 1.0 : 0.0;
      for (int k = c; k < i; ++k) s -= a[i * LP + k] * inv[k * LP + c];
      inv[i * LP + c] = s * dinv[i];
    }
  }
  __syncthreads();

  double* l = Lmat + (long long)b * sG + (long long)o * r + o;
  double* di_out = Dinv + (long long)b * sD;
  for (int e = tid; e < NB * NB; e += 256) {
    const int i = e / NB, j = e % NB;
    if (i < nb && j < nb) l[(long long)i * r + j] = j <= i ? a[i * LP + j] : 0.0;
    di_out[i * NB + j] = (i < nb && j <= i && j < nb) ? inv[i * LP + j] : 0.0;
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
