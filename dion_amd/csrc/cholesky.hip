// One block-column step of the batched, blocked Cholesky (fp64 or fp32) used by the CholeskyQR
// orthonormalisation, fused into a single launch: every workgroup factors the (<= 64) x (<= 64)
// diagonal block on the matrix cores and inverts the triangular factor (redundantly -- the factor is
// the serial part; a few workgroups per matrix repeat it rather than wait for one), then they share
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

// The 64 x 64 diagonal block S and the inverse-in-progress Y live in matrix-core accumulators: wavefront w of
// the four holds tile row w (rows 16 w .. 16 w + 15) of both as 16 x 16 tiles.  Right-looking with 4-wide block
// columns.  Per block step every wavefront reads the published block column of S (64 x 4) and row block of Y
// (4 x 64) from LDS and repeats the serial part on its own SIMD instead of waiting for one owner: the 4 x 4
// diagonal factor (the same instructions in every lane), then lane = row forms its row of the L block column
// by forward substitution and lane = column its column of X = L_cc^-1 Y_c (rows 4 cb .. 4 cb + 3 of the inverse,
// final after this).  Both go to LDS as MFMA operands, the two rank-4 updates S -= L_c L_c^T, Y -= L_c X are
// v_mfma_*_16x16x4 instructions on the wavefront's own tiles, and the wavefronts publish the next block column / row
// block.  One workgroup barrier per 4 columns; the published blocks and the operands are double-buffered.
template <typename T> __device__ __forceinline__ T rsqrt_seed(T p);
template <> __device__ __forceinline__ double rsqrt_seed<double>(double p) { return __builtin_amdgcn_rsq(p); }
template <> __device__ __forceinline__ float rsqrt_seed<float>(float p) { return __builtin_amdgcn_rsqf(p); }
// a positive normal number (false for NaN, infinities, zero and denormals, which the estimate does not handle)
__device__ __forceinline__ bool usable_pivot(double p) { return __builtin_amdgcn_class(p, 0x100); }
__device__ __forceinline__ bool usable_pivot(float p) { return __builtin_amdgcn_classf(p, 0x100); }

template <typename T> struct Quad { T v[4]; };

template <typename T>
__global__ __launch_bounds__(256) void chol_step_kernel(const T* __restrict__ G, T* __restrict__ Lmat,
                                                        T* __restrict__ Wmat, long long sG, int r, int o, int nb,
                                                        int below, int* __restrict__ info, int fresh, const int* gate,
                                                        int gate_want) {
  typedef typename Mfma<T>::acc_t acc_t;
  typedef Quad<T> quad_t;
  __shared__ __attribute__((aligned(16))) T scol[2][4][NB];     // published block column of S: [column][row]
  __shared__ __attribute__((aligned(16))) quad_t yrow[2][NB];   // published row block of Y:    [column] -> 4 rows
  __shared__ __attribute__((aligned(16))) quad_t lops[2][NB];   // L block column as MFMA operand (0 in finished rows)
  __shared__ __attribute__((aligned(16))) quad_t xops[2][NB];   // X, [column] -> 4 rows
  extern __shared__ __attribute__((aligned(16))) unsigned char opnd_raw[];   // two k-major 64 x 64 operand tiles
  T* const opnd = reinterpret_cast<T*>(opnd_raw);
  const int b = blockIdx.y, tid = threadIdx.x;
  if (gate && (gate[b] != 0) != (gate_want != 0)) return;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lc = lane & 15, lg = lane >> 4;
  // D_j transposed (dT[k][x] = D[x][k], zero outside the nb x nb lower triangle) and, for role 0, L_jj (in `op`)
  T* const dT = opnd;
  T* const op = opnd + NB * LP;
  const T* g = G + (long long)b * sG + (long long)o * r + o;
  acc_t S[4], Y[4];
#pragma unroll
  for (int tj = 0; tj < 4; ++tj)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int i = wave * 16 + Mfma<T>::row(v, lane), j = tj * 16 + lc;
      // identity padding beyond nb keeps the padded part inert
      S[tj][v] = (tj <= wave && i < nb && j < nb) ? g[(long long)i * r + j] : (i == j ? T(1) : T(0));
      Y[tj][v] = (i == j) ? T(1) : T(0);
    }
  // The workgroups of one matrix share its roles round-robin (role 0: L_jj, D_j and the status word; 1 .. below:
  // panel tiles; the rest: W tiles).  The operand tile of a product does not depend on this step's factor: it is
  // requested now, 16 elements per thread, and the next one while the previous product runs.
  const int nroles = 1 + below + o / NB;
  T pre[16];
  auto fetch = [&](int role) {
    const bool panel = role <= below;
    const int row0 = o + nb + (role - 1) * NB;
    const int rows_ok = r - row0 < NB ? r - row0 : NB;
    const T* src = panel ? G + (long long)b * sG + (long long)row0 * r + o
                         : Lmat + (long long)b * sG + (long long)o * r + (role - 1 - below) * NB;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int e = tid + 256 * t, hi = e >> 6, lo = e & 63;
      const bool in = panel ? (hi < rows_ok && lo < nb) : hi < nb;
      pre[t] = in ? src[(long long)hi * r + lo] : T(0);
    }
  };
  int role = blockIdx.x == 0 ? (int)gridDim.x : (int)blockIdx.x;   // this workgroup's first product
  if (role < nroles) fetch(role);
  if (tid < 2 * NB) {
    // columns right of the diagonal tile of a row block are never published: they read as zero
    quad_t z;
#pragma unroll
    for (int k = 0; k < 4; ++k) z.v[k] = T(0);
    yrow[tid >> 6][tid & 63] = z;
  }
  __syncthreads();

  // Block q (columns / rows 4 q .. 4 q + 3) of the current S and Y into buffer `buf`.
  auto publish = [&](int q, int buf) {
    const int tq = q >> 2, qq = q & 3;
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) {
      if (tj == tq && tj <= wave && (lc >> 2) == qq) {
#pragma unroll
        for (int v = 0; v < 4; ++v) scol[buf][lc & 3][wave * 16 + Mfma<T>::row(v, lane)] = S[tj][v];
      }
      if (wave == tq && tj <= wave) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int rr = Mfma<T>::row(v, lane);
          if ((rr >> 2) == qq) yrow[buf][tj * 16 + lc].v[rr & 3] = Y[tj][v];
        }
      }
    }
  };
  publish(0, 0);
  __syncthreads();

  constexpr int NEWTON = sizeof(T) == 8 ? 2 : 0;   // the hardware estimate is good to 1 ulp in fp32, ~2^-27 in fp64
  int bad = 0;                                     // first failed pivot (every lane computes the same)
  for (int cb = 0; cb < NB / 4; ++cb) {
    const int buf = cb & 1, k0 = cb * 4;
    quad_t sv;                             // lane = row: S[lane][k0 ..]
#pragma unroll
    for (int k = 0; k < 4; ++k) sv.v[k] = scol[buf][k][lane];
    const quad_t yv = yrow[buf][lane];     // lane = column: Y[k0 ..][lane]
    T a[4][4];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const quad_t d = *reinterpret_cast<const quad_t*>(&scol[buf][jj][k0]);   // the same address in every lane
#pragma unroll
      for (int ii = 0; ii < 4; ++ii) a[ii][jj] = d.v[ii];
    }
    // unblocked Cholesky of the 4 x 4 diagonal block: a[i][j], j < i becomes L_cc, di[] the inverse diagonal
    T di[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const T p = a[c][c];
      const bool ok = usable_pivot(p);
      // 1/sqrt(p) from the hardware estimate plus Newton steps: this chain is the critical path of the whole
      // factorisation and the library sqrt + divide are four times as long
      T rs = ok ? rsqrt_seed<T>(p) : T(0);
#pragma unroll
      for (int it = 0; it < NEWTON; ++it) rs = rs * (T(1.5) - T(0.5) * p * rs * rs);
      di[c] = ok ? rs : T(0);
      bad = (!ok && bad == 0 && k0 + c < nb) ? o + k0 + c + 1 : bad;
#pragma unroll
      for (int i = c + 1; i < 4; ++i) a[i][c] *= di[c];
#pragma unroll
      for (int i = c + 1; i < 4; ++i)
#pragma unroll
        for (int j = c + 1; j <= i; ++j) a[i][j] -= a[i][c] * a[j][c];
    }
    // row `lane` of the L block column and column `lane` of X, by forward substitution with L_cc
    T l[4], x[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      T tl = sv.v[k], tx = yv.v[k];
#pragma unroll
      for (int m = 0; m < k; ++m) {
        tl -= l[m] * a[k][m];
        tx -= a[k][m] * x[m];
      }
      l[k] = tl * di[k];
      x[k] = tx * di[k];
    }
    quad_t lo, xo, lfin;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      lo.v[k] = lane > k0 + 3 ? l[k] : T(0);               // finished rows take no part in the updates
      lfin.v[k] = lane >= k0 + k ? l[k] : T(0);            // L_jj: zero above the diagonal
      xo.v[k] = (lane <= k0 + k && k0 + k < nb) ? x[k] : T(0);
    }
    lops[buf][lane] = lo;     // (every wavefront writes the same values; each reads back after its own writes)
    xops[buf][lane] = xo;
    if (wave == (cb & 3)) {
#pragma unroll
      for (int k = 0; k < 4; ++k) dT[lane * LP + k0 + k] = lane < nb ? xo.v[k] : T(0);
      if (blockIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < 4; ++k) op[lane * LP + k0 + k] = lfin.v[k];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (wave * 16 + 15 > k0 + 3) {
      const T aop = -lops[buf][wave * 16 + lc].v[lg];
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) {
        if (tj <= wave && tj * 16 + 15 > k0 + 3) S[tj] = Mfma<T>::mma(aop, lops[buf][tj * 16 + lc].v[lg], S[tj]);
        if (tj <= wave && tj * 16 <= k0 + 3) Y[tj] = Mfma<T>::mma(aop, xops[buf][tj * 16 + lc].v[lg], Y[tj]);
      }
    }
    if (cb + 1 < NB / 4) publish(cb + 1, buf ^ 1);
    __syncthreads();
  }

  // ---- the 64 x 64 x 64 products that depend on the factor: C[m][n] = sum_k opa[k][m] * opb[k][n]
  if (blockIdx.x == 0) {
    T* l = Lmat + (long long)b * sG + (long long)o * r + o;
    T* w = Wmat + (long long)b * sG + (long long)o * r + o;
    for (int e = tid; e < NB * NB; e += 256) {
      const int i = e >> 6, j = e & 63;
      if (i < nb && j < nb) {
        l[(long long)i * r + j] = op[i * LP + j];
        w[(long long)i * r + j] = dT[j * LP + i];
      }
    }
    // (`fresh`: the first block column of a factorisation starts the matrix's status word)
    if (tid == 0 && (fresh || (bad != 0 && info[b] == 0))) info[b] = bad;
  }
  const int wm = wave >> 1, wn = wave & 1;
  while (role < nroles) {
    const bool panel = role <= below;
    __syncthreads();   // `op` may still be read (role 0's copy, the previous product's MFMAs)
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int e = tid + 256 * t;
      // panel: opa[k][m] = A[row0 + m][o + k] (element e = (m, k));  W: opb[k][n] = L[o + k][col0 + n] (e = (k, n))
      op[panel ? (e & 63) * LP + (e >> 6) : (e >> 6) * LP + (e & 63)] = pre[t];
    }
    const int next = role + (int)gridDim.x;
    if (next < nroles) fetch(next);   // in flight during this role's product
    __syncthreads();
    const int row0 = panel ? o + nb + (role - 1) * NB : o;
    const int col0 = panel ? o : (role - 1 - below) * NB;   // (W: col0 + 64 <= o)
    const int rows_ok = panel ? (r - row0 < NB ? r - row0 : NB) : nb;
    const int cols_ok = panel ? nb : NB;
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
    role = next;
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
