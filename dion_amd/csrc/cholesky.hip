// One block-column step of the batched, blocked fp64 Cholesky used by the CholeskyQR
// orthonormalisation, fused into a single launch: every workgroup factors the (<= 64) x (<= 64)
// diagonal block in registers and inverts the triangular factor (redundantly -- the factor is the
// serial part; a few workgroups per matrix repeat it rather than wait for one), then they share
// the 64 x 64 pieces of what depends on it:
//   role 0            : stores L_jj and its inverse D_j (the diagonal block of W, see below),
//   roles 1 .. below  : one 64-row tile of the panel   L[i, j] = A[i, j] D_j^T,
//   roles above that  : one 64-column tile of          W[j, c] = -D_j L[j, c],  c < j,
// where W is the block-lower-triangular matrix with which the triangular solve of P becomes one
// in-place GEMM per block column:  P[:, j] <- P[:, 0 .. j] W[j, 0 .. j]^T.
// No host synchronisation: a failed pivot is recorded in a device-side info word, mirroring
// torch.linalg.cholesky_ex's `info`.
#include "gemm_f64.h"

// fp64 factorisation: fused multiply-adds are welcome here (the build disables contraction
// globally for the kernels that reproduce the reference's bf16 rounding points)
#pragma clang fp contract(fast)

namespace {

constexpr int NB = DA_CHOL_NB;
constexpr int LP = NB + 1;   // LDS pitch of the operand tiles (doubles): transposed stores stay nearly conflict-free

// 256 threads as a 16 x 16 grid; thread (bi, bj) keeps the 4 x 4 blocks of the working matrix
// and of the inverse-in-progress at block position (bi, bj) in registers.  Right-looking with
// 4-wide block columns: per block step the diagonal owner factors and inverts its 4 x 4 block
// in registers, the column owners form their L blocks (A_ic * L_cc^-T), the row owners of the
// inverse form X_c = L_cc^-1 * Y_c, both are published through LDS, and every thread applies
// the two rank-4 updates.  Two barriers per 4 columns.
template <typename T> __device__ __forceinline__ T rsqrt_seed(T p);
template <> __device__ __forceinline__ double rsqrt_seed<double>(double p) { return __builtin_amdgcn_rsq(p); }
template <> __device__ __forceinline__ float rsqrt_seed<float>(float p) { return __builtin_amdgcn_rsqf(p); }

template <typename T>
__global__ __launch_bounds__(256) void chol_step_kernel(const T* __restrict__ G, T* __restrict__ Lmat,
                                                        T* __restrict__ Wmat, long long sG, int r, int o, int nb,
                                                        int below, int* __restrict__ info, int fresh, const int* gate,
                                                        int gate_want) {
  typedef typename Mfma<T>::acc_t acc_t;
  __shared__ T dinv4[4][4];            // inverse of the current diagonal 4 x 4 factor (lower)
  __shared__ T lcol[NB][4];            // rows > 4cb+3: L[i][4cb .. 4cb+3]
  __shared__ T xrow[4][NB];            // rows 4cb .. 4cb+3 of L^-1
  __shared__ int first_bad;
  extern __shared__ __attribute__((aligned(16))) unsigned char opnd_raw[];   // two k-major 64 x 64 operand tiles
  T* const opnd = reinterpret_cast<T*>(opnd_raw);
  const int b = blockIdx.y, tid = threadIdx.x;
  if (gate && (gate[b] != 0) != (gate_want != 0)) return;
  const int bi = tid >> 4, bj = tid & 15;
  const T* g = G + (long long)b * sG + (long long)o * r + o;
  T a[4][4], y[4][4];
#pragma unroll
  for (int ii = 0; ii < 4; ++ii)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int i = bi * 4 + ii, j = bj * 4 + jj;
      // identity padding beyond nb keeps the padded part inert
      a[ii][jj] = (i < nb && j < nb) ? g[(long long)i * r + j] : (i == j ? T(1) : T(0));
      y[ii][jj] = (i == j) ? T(1) : T(0);
    }
  if (tid == 0) first_bad = 0;
  __syncthreads();

  for (int cb = 0; cb < NB / 4; ++cb) {
    if (bi == cb && bj == cb) {
      // unblocked Cholesky of the 4 x 4 diagonal block and its inverse, in registers
      T di[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const T p = a[c][c];
        const bool ok = p > T(0) && p < (sizeof(T) == 8 ? T(1.0e300) : T(1.0e37));  // false for NaN as well
        // 1/sqrt(p) from the hardware estimate plus two Newton steps (full fp64 accuracy), then
        // sqrt(p) = p * rsqrt(p): this thread is the critical path of the whole factorisation and
        // the library sqrt + divide are four times as long
        T rs = ok ? rsqrt_seed<T>(p) : T(0);
        rs = rs * (T(1.5) - T(0.5) * p * rs * rs);
        rs = rs * (T(1.5) - T(0.5) * p * rs * rs);
        const T d = ok ? p * rs : T(0);
        di[c] = ok ? rs : T(0);
        if (!ok && cb * 4 + c < nb && first_bad == 0) first_bad = o + cb * 4 + c + 1;
        a[c][c] = d;
#pragma unroll
        for (int i = c + 1; i < 4; ++i) a[i][c] *= di[c];
#pragma unroll
        for (int i = c + 1; i < 4; ++i)
#pragma unroll
          for (int j = c + 1; j <= i; ++j) a[i][j] -= a[i][c] * a[j][c];
      }
      T inv[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          T t = (i == j) ? T(1) : T(0);
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (k >= j && k < i) t -= a[i][k] * inv[k][j];
          inv[i][j] = j <= i ? t * di[i] : T(0);
        }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (j > i) a[i][j] = T(0);
          dinv4[i][j] = inv[i][j];
        }
    }
    __syncthreads();
    if (bj == cb && bi > cb) {
      // L_ic = A_ic * L_cc^-T : row ii of the block times the transposed inverse
      T l[4][4];
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          T t = T(0);
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
      T x[4][4];
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          T t = T(0);
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
      T li[4][4];
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int k = 0; k < 4; ++k) li[ii][k] = lcol[bi * 4 + ii][k];
      if (bj > cb) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const T lj = lcol[bj * 4 + jj][k];
#pragma unroll
            for (int ii = 0; ii < 4; ++ii) a[ii][jj] -= li[ii][k] * lj;
          }
      }
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const T xk = xrow[k][bj * 4 + jj];
#pragma unroll
          for (int ii = 0; ii < 4; ++ii) y[ii][jj] -= li[ii][k] * xk;
        }
    }
  }

  // D_j (zero outside its nb x nb lower triangle), transposed: dT[k][x] = D[x][k]
  T* dT = opnd;
  T* op = opnd + NB * LP;
#pragma unroll
  for (int ii = 0; ii < 4; ++ii)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int i = bi * 4 + ii, j = bj * 4 + jj;
      dT[j * LP + i] = (i < nb && j <= i) ? y[ii][jj] : T(0);
    }
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int nroles = 1 + below + o / NB;
  // the workgroups of one matrix share its roles round-robin
  for (int role = blockIdx.x; role < nroles; role += gridDim.x) {
    if (role == 0) {
      T* l = Lmat + (long long)b * sG + (long long)o * r + o;
      T* w = Wmat + (long long)b * sG + (long long)o * r + o;
#pragma unroll
      for (int ii = 0; ii < 4; ++ii)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int i = bi * 4 + ii, j = bj * 4 + jj;
          if (i < nb && j < nb) {
            l[(long long)i * r + j] = j <= i ? a[ii][jj] : T(0);
            w[(long long)i * r + j] = j <= i ? y[ii][jj] : T(0);
          }
        }
      // (`fresh`: the first block column of a factorisation starts the matrix's status word)
      if (tid == 0 && (fresh || (first_bad != 0 && info[b] == 0))) info[b] = first_bad;
      continue;
    }
    // 64 x 64 x 64 product on the matrix cores: C[m][n] = sum_k opa[k][m] * opb[k][n]
    const bool panel = role <= below;
    int row0, col0, rows_ok, cols_ok;
    __syncthreads();   // `op` may still be read by the previous role's MFMAs; dT is complete after it
    if (panel) {
      // L[i, j] = A[i, j] D^T :  opa[k][m] = A[row0 + m][o + k],  opb = dT
      row0 = o + nb + (role - 1) * NB;
      col0 = o;
      rows_ok = r - row0 < NB ? r - row0 : NB;
      cols_ok = nb;
      const T* src = G + (long long)b * sG + (long long)row0 * r + o;
      for (int e = tid; e < NB * NB; e += 256) {
        const int m = e >> 6, k = e & 63;
        op[k * LP + m] = (m < rows_ok && k < nb) ? src[(long long)m * r + k] : T(0);
      }
    } else {
      // W[j, c] = -D L[j, c] :  opa = dT,  opb[k][n] = L[o + k][col0 + n]
      row0 = o;
      col0 = (role - 1 - below) * NB;   // col0 + 64 <= o
      rows_ok = nb;
      cols_ok = NB;
      const T* src = Lmat + (long long)b * sG + (long long)o * r + col0;
      for (int e = tid; e < NB * NB; e += 256) {
        const int k = e >> 6, n = e & 63;
        op[k * LP + n] = k < nb ? src[(long long)k * r + n] : T(0);
      }
    }
    __syncthreads();
    const T* opa = panel ? op : dT;
    const T* opb = panel ? dT : op;
    acc_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = acc_t{0, 0, 0, 0};
#pragma unroll 4
    for (int ks = 0; ks < NB / 4; ++ks) {
      const int k = ks * 4 + (lane >> 4);
      T af[2], bfv[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = opa[k * LP + wm * 32 + i * 16 + (lane & 15)];
#pragma unroll
      for (int j = 0; j < 2; ++j) bfv[j] = opb[k * LP + wn * 32 + j * 16 + (lane & 15)];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = Mfma<T>::mma(af[i], bfv[j], acc[i][j]);
    }
    T* dst = (panel ? Lmat : Wmat) + (long long)b * sG + (long long)row0 * r + col0;
    const T sign = panel ? T(1) : T(-1);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = wm * 32 + i * 16 + Mfma<T>::row(v, lane);
          const int n = wn * 32 + j * 16 + (lane & 15);
          if (m < rows_ok && n < cols_ok) dst[(long long)m * r + n] = sign * acc[i][j][v];
        }
  }
}

template <typename T>
int chol_step(const T* G, T* Lmat, T* Wmat, long long sG, int r, int o, int nb, int* info, int batch, DaGate gate,
              bool fresh, hipStream_t s) {
  if (nb <= 0 || nb > NB || o < 0 || o + nb > r || (o % NB) != 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  const int rest = r - o - nb;
  if (rest > 0 && nb != NB) return DA_ERR_ARG;
  const int below = (rest + NB - 1) / NB;
  const int smem = 2 * NB * LP * (int)sizeof(T);
  // workgroups per matrix: as many as fit one per CU over the batch (the factorisation every workgroup repeats is
  // bound by fp64 instruction issue, which two workgroups on a CU would share: 384 instead of 256 in flight cost
  // 3 % of the orthonormaliser on a 48-matrix bucket), never more than there are roles
  const int nroles = 1 + below + o / NB;
  int per = 256 / batch;
  if (per < 1) per = 1;
  if (per > nroles) per = nroles;
  static bool configured = false;  // benign race: the attribute call is idempotent
  if (!configured) {
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(chol_step_kernel<T>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    configured = true;
  }
  hipLaunchKernelGGL(chol_step_kernel<T>, dim3(per, batch), dim3(256), smem, s, G, Lmat, Wmat, sG, r, o, nb, below, info,
                     fresh ? 1 : 0, gate.flags, gate.want);
  return da_launch_status();
}

}  // namespace

int da_chol_step(const double* G, double* Lmat, double* Wmat, long long sG, int r, int o, int nb, int* info,
                 int batch, DaGate gate, hipStream_t s) {
  return chol_step<double>(G, Lmat, Wmat, sG, r, o, nb, info, batch, gate, false, s);
}
int da_chol_step_f32(const float* G, float* Lmat, float* Wmat, long long sG, int r, int o, int nb, int* info,
                     int batch, DaGate gate, hipStream_t s) {
  // the fp32 pass keeps its status in a word of its own, which its first block column initialises
  return chol_step<float>(G, Lmat, Wmat, sG, r, o, nb, info, batch, gate, o == 0, s);
}
