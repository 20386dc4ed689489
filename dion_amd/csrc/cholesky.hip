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
// A second form of the kernel (INV) writes, instead of W's row block, row block j of T = L^-1 itself:
//   T[j, j] = D_j,   T[j, c] = -D_j sum_{k = c .. j-1} L[j, k] T[k, c],   c < j,
// for the callers that need the inverse factor as a matrix.
// Deferred trailing update (o_prev >= 0): the rank-64 update of the previous step, A[i, c] -= L[i, p] L[c, p]^T
// (p = the previous block column), has not been applied to the matrix.  This launch applies it where it needs it
// -- every workgroup to the diagonal block before factoring it, a panel role to its tile -- and further workgroups
// (workgroup index >= per) do nothing but apply it to the tiles right of this block column (up to column c_end), which
// the later steps read: the separate update launch between two steps is gone.
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

template <typename T, bool INV>
__global__ __launch_bounds__(256) void chol_step_kernel(T* __restrict__ G, T* __restrict__ Lmat,
                                                        T* __restrict__ Wmat, T* __restrict__ Tmat, long long sG, int r,
                                                        int o, int nb, int below, int* __restrict__ info, int fresh,
                                                        const int* gate, int gate_want, int o_prev, int c_end, int per, int t_row, int n_t,
                                                        int t_inline, T* __restrict__ pstat) {
  typedef typename Mfma<T>::acc_t acc_t;
  typedef Quad<T> quad_t;
  __shared__ __attribute__((aligned(16))) T scol[2][4][NB];     // published block column of S: [column][row]
  __shared__ __attribute__((aligned(16))) quad_t yrow[2][NB];   // published row block of Y:    [column] -> 4 rows
  __shared__ __attribute__((aligned(16))) quad_t lops[2][NB];   // L block column as MFMA operand (0 in finished rows)
  __shared__ __attribute__((aligned(16))) quad_t xops[2][NB];   // X, [column] -> 4 rows
  extern __shared__ __attribute__((aligned(16))) unsigned char opnd_raw[];   // two k-major 64 x 64 operand tiles
  T* const opnd = reinterpret_cast<T*>(opnd_raw);
  // grid (matrix, workgroup of the matrix): the matrices' workgroups 0 are dispatched first, the update-only
  // workgroups of a deferred trailing update last -- they must not keep the serial part waiting for a CU
  const int b = blockIdx.x, wg = blockIdx.y, tid = threadIdx.x;
  if (gate && (gate[b] != 0) != (gate_want != 0)) return;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lc = lane & 15, lg = lane >> 4;
  // D_j transposed (dT[k][x] = D[x][k], zero outside the nb x nb lower triangle) and, for role 0, L_jj (in `op`)
  T* const dT = opnd;
  T* const op = opnd + NB * LP;
  // deferred mode: L[j, p] k-major (ljT[k][n] = L[o + n][o_prev + k]), behind the role buffers
  T* const ljT = opnd + (INV ? 5 : 2) * NB * LP;
  const bool defer = o_prev >= 0;
  const T* g = G + (long long)b * sG + (long long)o * r + o;
  // The workgroups of one matrix share its roles round-robin (role 0: L_jj, D_j and the status word; 1 .. below:
  // panel tiles; the rest: W tiles).  The operand tile of a product does not depend on this step's factor: it is
  // requested now, 16 elements per thread, and the next one while the previous product runs.
  const int nroles = 1 + below + ((!INV || t_inline) ? o / NB : 0);
  // row block of T that the T roles work on: this step's, or an earlier one in the workgroups that only do that
  int t_o = o, t_nb = nb;
  // A 64 x 64 tile in registers: thread t holds the four elements (row (t >> 4) + 16 q, columns 4 (t & 15) .. + 3),
  // q = 0 .. 3 (named vectors, not an array: an array that one loop iteration writes and the next one reads ends up
  // in scratch memory).
  typedef T tv4_t __attribute__((ext_vector_type(4)));
  const tv4_t tz = {T(0), T(0), T(0), T(0)};
  tv4_t pa0 = tz, pa1 = tz, pa2 = tz, pa3 = tz, pb0 = tz, pb1 = tz, pb2 = tz, pb3 = tz;
  const int trow = tid >> 4, tcol = (tid & 15) * 4;
  // rows < rows_ok, columns < cols_ok of the tile at src (row pitch r); the rest reads as zero
  auto load_quad = [&](const T* src, int q, int rows_ok, int cols_ok) __attribute__((always_inline)) {
    const int row = trow + 16 * q;
    tv4_t v = {T(0), T(0), T(0), T(0)};
    if (row < rows_ok) {
      const T* p = src + (long long)row * r + tcol;
      if (tcol + 4 <= cols_ok) {
        v = *reinterpret_cast<const tv4_t*>(p);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = tcol + i < cols_ok ? p[i] : T(0);
      }
    }
    return v;
  };
#define DA_LOAD_TILE(v0, v1, v2, v3, src, rows_ok, cols_ok)                                  \
  do {                                                                                       \
    v0 = load_quad((src), 0, (rows_ok), (cols_ok)); v1 = load_quad((src), 1, (rows_ok), (cols_ok)); \
    v2 = load_quad((src), 2, (rows_ok), (cols_ok)); v3 = load_quad((src), 3, (rows_ok), (cols_ok)); \
  } while (0)
  // quad -> LDS tile, k-major with pitch LP: transposed (element (row, col) at [col][row]) or as it is
  auto store_quad = [&](const tv4_t v, int q, T* dst, bool transposed) __attribute__((always_inline)) {
    const int row = trow + 16 * q;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (transposed) dst[(tcol + i) * LP + row] = v[i];
      else dst[row * LP + tcol + i] = v[i];
    }
  };
#define DA_STORE_TILE(v0, v1, v2, v3, dst, transposed)                                       \
  do {                                                                                       \
    store_quad(v0, 0, (dst), (transposed)); store_quad(v1, 1, (dst), (transposed));          \
    store_quad(v2, 2, (dst), (transposed)); store_quad(v3, 3, (dst), (transposed));          \
  } while (0)
  const int wm = wave >> 1, wn = wave & 1;
  // acc += opa^T opb over one 64-deep tile pair (k-major tiles of pitch LP)
  auto mma_tile = [&](const T* opa, const T* opb, acc_t (&acc)[2][2]) __attribute__((always_inline)) {
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
        for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::mma(af[i], bfv[j], acc[i][j]);
    }
  };
  // operand tiles of one term of T[j, c] = -D_j sum_{k = c .. j-1} L[j, k] T[k, c]  (j = o / 64): L[j, k] and T[k, c]
  auto fetch_t = [&](int c, int k) __attribute__((always_inline)) {
    if (!INV) return;
    DA_LOAD_TILE(pa0, pa1, pa2, pa3, Lmat + (long long)b * sG + (long long)t_o * r + (long long)k * NB, t_nb, NB);
    DA_LOAD_TILE(pb0, pb1, pb2, pb3, Tmat + (long long)b * sG + (long long)k * NB * r + (long long)c * NB, NB, NB);
  };
  // Row block jb (rows t_o ..) of T = L^-1, column block c:  T[jb, c] = -D sum_{k = c .. jb-1} L[jb, k] T[k, c]  with
  // D (transposed, in dT) the inverse of the row's diagonal block.  `have_first`: the first tile pair is already in
  // the registers; next_role >= 0: that role's operand is requested before the last product.
  auto t_tile = [&](int c, int jb, bool have_first, int next_role, auto fetch_next) __attribute__((always_inline)) {
      acc_t acc[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = acc_t{0, 0, 0, 0};
      // the tile pairs alternate between two LDS buffers: pair k + 1 is requested before the product of pair k and
      // written after it (the registers live within one iteration)
      auto put = [&](int buf) __attribute__((always_inline)) {
        T* pa = op + buf * (2 * NB * LP);
        DA_STORE_TILE(pa0, pa1, pa2, pa3, pa, true);              // opa[kk][m] = L[t_o + m][64 k + kk]
        DA_STORE_TILE(pb0, pb1, pb2, pb3, pa + NB * LP, false);  // opb[kk][n] = T[64 k + kk][64 c + n]
      };
      if (!have_first) fetch_t(c, c);
      __syncthreads();   // the buffers may still be read (role 0's copy, a previous product)
      put(0);
      for (int k = c; k < jb; ++k) {
        const int buf = (k - c) & 1;
        if (k + 1 < jb) fetch_t(c, k + 1);
        __syncthreads();                                     // pair k is in place; the other buffer is free
        mma_tile(op + buf * (2 * NB * LP), op + buf * (2 * NB * LP) + NB * LP, acc);
        if (k + 1 < jb) put(buf ^ 1);
      }
      if (next_role >= 0) fetch_next(next_role);
      T* const op2 = op + NB * LP;   // (buffer 0's second tile: free after the barrier below)
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v)
            op2[(wm * 32 + i * 16 + Mfma<T>::row(v, lane)) * LP + wn * 32 + j * 16 + (lane & 15)] = acc[i][j][v];
      __syncthreads();
      acc_t res[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) res[i][j] = acc_t{0, 0, 0, 0};
      mma_tile(dT, op2, res);
      T* dst = Tmat + (long long)b * sG + (long long)t_o * r + (long long)c * NB;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int m = wm * 32 + i * 16 + Mfma<T>::row(v, lane);
            const int n = wn * 32 + j * 16 + (lane & 15);
            if (m < t_nb) dst[(long long)m * r + n] = -res[i][j][v];
          }
  };
  if (INV && wg >= per && wg < per + n_t) {
    // ---- rows of T only: block row t_row (a row whose diagonal block an earlier launch inverted), column blocks
    // wg - per, + n_t, ...; its inverse diagonal block comes from Tmat
    t_o = t_row * NB;
    t_nb = r - t_o < NB ? r - t_o : NB;
    {
      tv4_t d0, d1, d2, d3;
      DA_LOAD_TILE(d0, d1, d2, d3, Tmat + (long long)b * sG + (long long)t_o * r + t_o, t_nb, t_nb);
      DA_STORE_TILE(d0, d1, d2, d3, dT, true);   // dT[k][x] = D[x][k]
    }
    for (int c = wg - per; c < t_row; c += n_t) t_tile(c, t_row, false, -1, [](int) {});
    return;
  }
  if (wg >= per) {
    // ---- deferred trailing update only: tiles (ti, tc) of the lower triangle right of this block column, columns
    // below c_end:  A[ti, tc] -= L[ti, p] L[tc, p]^T
    const int jb = o / NB, nblk = (r + NB - 1) / NB, cblk = (c_end + NB - 1) / NB;
    int u = wg - per - n_t;
    const int stride = (int)gridDim.y - per - n_t;
    int tc = jb + 1, left = nblk - tc;   // tiles of column block tc: row blocks tc .. nblk - 1
    while (tc < cblk) {
      if (u >= left) { u -= left; ++tc; --left; continue; }
      const int ti = tc + u;
      const int rows_ok = r - ti * NB < NB ? r - ti * NB : NB;
      const int cols_ok = c_end - tc * NB < NB ? c_end - tc * NB : NB;
      const int crow_ok = r - tc * NB < NB ? r - tc * NB : NB;
      const T* lbase = Lmat + (long long)b * sG + o_prev;
      tv4_t ua0, ua1, ua2, ua3, ub0, ub1, ub2, ub3;   // (of this iteration only)
      DA_LOAD_TILE(ua0, ua1, ua2, ua3, lbase + (long long)ti * NB * r, rows_ok, NB);
      DA_LOAD_TILE(ub0, ub1, ub2, ub3, lbase + (long long)tc * NB * r, crow_ok, NB);
      __syncthreads();   // the previous tile's products are done with the buffers
      DA_STORE_TILE(ua0, ua1, ua2, ua3, dT, true);   // opa[k][m] = L[ti, p][m][k]
      DA_STORE_TILE(ub0, ub1, ub2, ub3, op, true);   // opb[k][n] = L[tc, p][n][k]
      __syncthreads();
      acc_t acc[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = acc_t{0, 0, 0, 0};
      mma_tile(dT, op, acc);
      T* dst = G + (long long)b * sG + (long long)ti * NB * r + (long long)tc * NB;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int m = wm * 32 + i * 16 + Mfma<T>::row(v, lane);
            const int n = wn * 32 + j * 16 + (lane & 15);
            if (m < rows_ok && n < cols_ok) dst[(long long)m * r + n] -= acc[i][j][v];
          }
      u += stride;
    }
    return;
  }
  if (defer) {
    // L[j, p], k-major: the deferred update of the diagonal block below and of this workgroup's panel tiles
    tv4_t lj0, lj1, lj2, lj3;
    DA_LOAD_TILE(lj0, lj1, lj2, lj3, Lmat + (long long)b * sG + (long long)o * r + o_prev, nb, NB);
    DA_STORE_TILE(lj0, lj1, lj2, lj3, ljT, true);
  }
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
  if (defer) {
    __syncthreads();   // ljT is in place
    // S -= L[j, p] L[j, p]^T on the wavefront's tile row (rows >= nb of ljT are zero: the padding stays inert)
#pragma unroll 4
    for (int ks = 0; ks < NB / 4; ++ks) {
      const T* lk = ljT + (ks * 4 + lg) * LP;
      const T aop = -lk[wave * 16 + lc];
#pragma unroll
      for (int tj = 0; tj < 4; ++tj)
        if (tj <= wave) S[tj] = Mfma<T>::mma(aop, lk[tj * 16 + lc], S[tj]);
    }
  }
  auto fetch = [&](int role) __attribute__((always_inline)) {
    const bool panel = role <= below;
    if (INV && !panel) {
      fetch_t(role - 1 - below, role - 1 - below);
      return;
    }
    const int row0 = o + nb + (role - 1) * NB;
    if (panel) {
      DA_LOAD_TILE(pa0, pa1, pa2, pa3, G + (long long)b * sG + (long long)row0 * r + o, r - row0 < NB ? r - row0 : NB, nb);
      // (deferred update: L[i, p] as well)
      if (defer) DA_LOAD_TILE(pb0, pb1, pb2, pb3, Lmat + (long long)b * sG + (long long)row0 * r + o_prev, r - row0 < NB ? r - row0 : NB, NB);
    } else DA_LOAD_TILE(pa0, pa1, pa2, pa3, Lmat + (long long)b * sG + (long long)o * r + (role - 1 - below) * NB, nb, NB);
  };
  int role = wg == 0 ? per : wg;   // this workgroup's first product (`per` workgroups share the roles)
  // (the two tiles of a T role would stay in registers through the whole factor loop: those are requested after it)
  const bool early = role < nroles && !(INV && role > below);
  if (early) fetch(role);
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
  T pmin = T(3e38), pmax = T(0);                   // smallest and largest usable pivot of this block column
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
      if (ok && k0 + c < nb) {
        pmin = p < pmin ? p : pmin;
        pmax = p > pmax ? p : pmax;
      }
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
      if (wg == 0) {
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
  if (wg == 0) {
    T* l = Lmat + (long long)b * sG + (long long)o * r + o;
    T* w = (INV ? Tmat : Wmat) + (long long)b * sG + (long long)o * r + o;
    for (int e = tid; e < NB * NB; e += 256) {
      const int i = e >> 6, j = e & 63;
      if (i < nb && j < nb) {
        l[(long long)i * r + j] = op[i * LP + j];
        w[(long long)i * r + j] = dT[j * LP + i];
      }
    }
    // (`fresh`: the first block column of a factorisation starts the matrix's status word)
    if (tid == 0 && (fresh || (bad != 0 && info[b] == 0))) info[b] = bad;
    // pivot range of the matrix so far (the squares of R's diagonal: their ratio bounds cond(R)^2 from below)
    if (tid == 0 && pstat) {
      T mn = pmin, mx = pmax;
      if (o > 0) {
        mn = pstat[2 * b] < mn ? pstat[2 * b] : mn;
        mx = pstat[2 * b + 1] > mx ? pstat[2 * b + 1] : mx;
      }
      pstat[2 * b] = mn;
      pstat[2 * b + 1] = mx;
    }
  }
  if (role < nroles && !early) fetch(role);
  while (role < nroles) {
    const bool panel = role <= below;
    if (INV && !panel) {
      const int next = role + per;
      t_tile(role - 1 - below, o / NB, true, next < nroles ? next : -1, fetch);
      role = next;
      continue;
    }
    if (defer && panel) {
      // the deferred update of this tile first:  A[i, j] -= L[i, p] L[j, p]^T
      __syncthreads();                                 // `op` may still be read
      DA_STORE_TILE(pb0, pb1, pb2, pb3, op, true);     // opa[k][m] = L[i, p][m][k]
      __syncthreads();
      acc_t du[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) du[i][j] = acc_t{0, 0, 0, 0};
      mma_tile(op, ljT, du);
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v)
            op[(wm * 32 + i * 16 + Mfma<T>::row(v, lane)) * LP + wn * 32 + j * 16 + (lane & 15)] = du[i][j][v];
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pa0[i] -= op[(trow + 0) * LP + tcol + i];
        pa1[i] -= op[(trow + 16) * LP + tcol + i];
        pa2[i] -= op[(trow + 32) * LP + tcol + i];
        pa3[i] -= op[(trow + 48) * LP + tcol + i];
      }
    }
    __syncthreads();   // `op` may still be read (role 0's copy, the previous product's MFMAs)
    // panel: opa[k][m] = A[row0 + m][o + k];  W: opb[k][n] = L[o + k][col0 + n]
    DA_STORE_TILE(pa0, pa1, pa2, pa3, op, panel);
    const int next = role + per;
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
    mma_tile(opa, opb, acc);
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

#undef DA_LOAD_TILE
#undef DA_STORE_TILE

template <typename T, bool INV>
int chol_step(T* G, T* Lmat, T* Wmat, T* Tmat, long long sG, int r, int o, int nb, int* info, int batch,
              DaGate gate, bool fresh, int o_prev, int c_end, int t_row, int t_inline, T* pstat, hipStream_t s) {
  if (nb <= 0 || nb > NB || o < 0 || o + nb > r || (o % NB) != 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  if (o_prev >= 0 && (o_prev != o - NB || c_end < o + nb || c_end > r)) return DA_ERR_ARG;
  const int rest = r - o - nb;
  if (rest > 0 && nb != NB) return DA_ERR_ARG;
  const int below = (rest + NB - 1) / NB;
  const int smem = ((INV ? 5 : 2) + 1) * NB * LP * (int)sizeof(T);   // (+ the tile of the deferred update)
  // workgroups per matrix: as many as fit one per CU over the batch (the factorisation every workgroup repeats is
  // bound by fp64 instruction issue, which two workgroups on a CU would share: 384 instead of 256 in flight cost
  // 3 % of the orthonormaliser on a 48-matrix bucket), never more than there are roles
  const int nroles = 1 + below + ((!INV || t_inline) ? o / NB : 0);
  if (t_row >= 0 && (!INV || t_row < 1 || t_row * NB >= o)) return DA_ERR_ARG;   // an earlier row with tiles left of its diagonal
  int per = 256 / batch;
  if (per < 1) per = 1;
  if (per > nroles) per = nroles;
  static DaOncePerDevice configured;
  const int rc_cfg = configured.run([&]() -> int {
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(chol_step_kernel<T, INV>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return DA_OK;
  });
  if (rc_cfg) return rc_cfg;
  // update-only workgroups of a deferred trailing update: one per tile right of this block column (columns below
  // c_end, lower triangle), at most 1024 over the batch
  int extra = 0;
  if (o_prev >= 0) {
    const int jb = o / NB, nblk = (r + NB - 1) / NB, cblk = (c_end + NB - 1) / NB;
    long long tiles = 0;
    for (int tc = jb + 1; tc < cblk; ++tc) tiles += nblk - tc;
    const long long cap = 1024 / batch > 1 ? 1024 / batch : 1;
    extra = (int)(tiles < cap ? tiles : cap);
  }
  // workgroups for the row of T that lags behind: one per tile of the row, at most 512 over the batch
  int n_t = 0;
  if (t_row >= 1) {
    const int cap = 512 / batch > 1 ? 512 / batch : 1;
    n_t = t_row < cap ? t_row : cap;
  }
  hipLaunchKernelGGL((chol_step_kernel<T, INV>), dim3(batch, per + n_t + extra), dim3(256), smem, s, G, Lmat, Wmat, Tmat, sG, r,
                     o, nb, below, info, fresh ? 1 : 0, gate.flags, gate.want, o_prev, c_end, per, t_row, n_t, t_inline, pstat);
  return da_launch_status();
}

}  // namespace

int da_chol_step(double* G, double* Lmat, double* Wmat, long long sG, int r, int o, int nb, int* info,
                 int batch, DaGate gate, hipStream_t s, int o_prev, int c_end, double* pstat) {
  return chol_step<double, false>(G, Lmat, Wmat, nullptr, sG, r, o, nb, info, batch, gate, false, o_prev, c_end, -1, 1, pstat, s);
}
int da_chol_step_f32(float* G, float* Lmat, float* Wmat, long long sG, int r, int o, int nb, int* info,
                     int batch, DaGate gate, hipStream_t s, int o_prev, int c_end) {
  // the fp32 pass keeps its status in a word of its own, which its first block column initialises
  return chol_step<float, false>(G, Lmat, Wmat, nullptr, sG, r, o, nb, info, batch, gate, o == 0, o_prev, c_end, -1, 1, nullptr, s);
}
int da_chol_step_f32_inv(float* G, float* Lmat, float* Tmat, long long sG, int r, int o, int nb, int* info,
                         int batch, DaGate gate, hipStream_t s, int o_prev, int c_end, int t_row, int t_inline) {
  return chol_step<float, true>(G, Lmat, nullptr, Tmat, sG, r, o, nb, info, batch, gate, o == 0, o_prev, c_end, t_row,
                                t_inline, nullptr, s);
}
int da_chol_trow_f32(float* Lmat, float* Tmat, long long sG, int r, int t_row, int batch, DaGate gate, hipStream_t s) {
  if (t_row < 1 || t_row * NB >= r || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  const int smem = 6 * NB * LP * (int)sizeof(float);
  const int cap = 512 / batch > 1 ? 512 / batch : 1;
  const int n_t = t_row < cap ? t_row : cap;
  // (the attribute is set by the first factorisation step, which always precedes this launch)
  hipLaunchKernelGGL((chol_step_kernel<float, true>), dim3(batch, n_t), dim3(256), smem, s, static_cast<float*>(nullptr), Lmat,
                     static_cast<float*>(nullptr), Tmat, sG, r, t_row * NB, r - t_row * NB < NB ? r - t_row * NB : NB, 0,
                     static_cast<int*>(nullptr), 0, gate.flags, gate.want, -1, 0, 0, t_row, n_t, 0, static_cast<float*>(nullptr));
  return da_launch_status();
}
