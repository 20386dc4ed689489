// Batched fp64 GEMM on the matrix cores (v_mfma_f64_16x16x4_f64) for the CholeskyQR
// orthonormalisation of Dion's P factor: the r x r Gram matrix P^T P (its condition number
// is the square of P's, hence fp64), the blocked Cholesky's panel / trailing updates and
// the blocked triangular solve P R^-1.
//
//   C[b] (M x N) = alpha * sum_k Aop[b](i,k) * Bop[b](j,k) + beta * E[b]
//
// 256 threads (2 x 2 wavefronts) per 64 x 64 tile, 16 k per stage; each wavefront owns
// 32 x 32 as 2 x 2 accumulators of 16 x 16.  LDS tiles are k-major [16][64] doubles for
// either operand layout, so the one-double-per-lane MFMA operands are conflict-free reads.
// Double buffered: the global loads of the next stage are in flight during the MFMAs.
// The same template is instantiated for fp32 (v_mfma_f32_16x16x4_f32; the polishing passes); the
// result may be stored as fp32 or bf16, and a block-triangular B operand shortens the sum per
// column tile.
#include "gemm_f64.h"

namespace {

constexpr int BK = 16;

template <bool KS, typename T>
__device__ __forceinline__ void fetch(T (&v)[4], const T* __restrict__ base, int ld, int row0, int k0,
                                      int rows, int K, int tid) {
  // the thread's 4 elements are contiguous in memory in either layout
  const int outer = KS ? k0 + (tid >> 4) : row0 + (tid >> 2);
  const int inner = KS ? row0 + (tid & 15) * 4 : k0 + (tid & 3) * 4;
  const int outer_n = KS ? K : rows, inner_n = KS ? rows : K;
  const T* p = base + (long long)outer * ld + inner;
  if (outer < outer_n && inner + 3 < inner_n && ((reinterpret_cast<uintptr_t>(p) & (2 * sizeof(T) - 1)) == 0)) {
    typedef T pair_t __attribute__((ext_vector_type(2)));   // 16 bytes (fp64) / 8 (fp32) / 4 (bf16) per access
    const pair_t lo = *reinterpret_cast<const pair_t*>(p);
    const pair_t hi = *reinterpret_cast<const pair_t*>(p + 2);
    v[0] = lo.x; v[1] = lo.y; v[2] = hi.x; v[3] = hi.y;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (outer < outer_n && inner + e < inner_n) ? p[e] : T(0);
  }
}

// Interior tiles (all rows and k in range, 16-byte aligned rows): the same four elements with no checks.
template <typename T>
__device__ __forceinline__ void fetch_fast(T (&v)[4], const T* __restrict__ p) {
  typedef T pair_t __attribute__((ext_vector_type(2)));
  const pair_t lo = *reinterpret_cast<const pair_t*>(p);
  const pair_t hi = *reinterpret_cast<const pair_t*>(p + 2);
  v[0] = lo.x; v[1] = lo.y; v[2] = hi.x; v[3] = hi.y;
}

// One 64-row slice of a stage goes to the k-major LDS tile lds[k][row] (row pitch BTt).
template <bool KS, int BTt, typename T>
__device__ __forceinline__ void put(T* lds, const T (&v)[4], int tid) {
  if (!KS) {
    const int r = tid >> 2, k4 = (tid & 3) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) lds[(k4 + e) * BTt + r] = v[e];
  } else {
    const int k = tid >> 4, r4 = (tid & 15) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) lds[k * BTt + r4 + e] = v[e];
  }
}

// BTt x BTt output tile, 256 threads as 2 x 2 wavefronts of (BTt / 2) x (BTt / 2) each.
template <typename T, bool A_KS, bool B_KS, bool SYM, int BTt>
__global__ __launch_bounds__(256) void gemm_f64_kernel(RealGemmDesc<T> d) {
  typedef typename Mfma<T>::acc_t acc_t;
  constexpr int H = BTt / 64;        // 64-row slices per operand stage
  constexpr int WT = BTt / 2;        // wavefront tile
  constexpr int TI = WT / 16;        // 16 x 16 accumulators per wavefront and direction
  __shared__ T lds_a[2][BK * BTt];
  __shared__ T lds_b[2][BK * BTt];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (d.M + BTt - 1) / BTt, tiles_n = (d.N + BTt - 1) / BTt;
  const bool tri = SYM || d.lower_only;
  // SYM: M == N; lower_only: M >= N, column tile c holds the tiles_m - c row tiles from the diagonal down
  const int per_batch = tri ? tiles_n * tiles_m - tiles_n * (tiles_n - 1) / 2 : tiles_m * tiles_n;
  const int split = blockIdx.y;  // split-K slice
  const int b = blockIdx.x / per_batch;
  if (d.gate && (d.gate[b] != 0) != (d.gate_want != 0)) return;
  int t = blockIdx.x - b * per_batch;
  int ti, tj;
  if (tri) {
    ti = 0;
    int len = tiles_m;
    while (t >= len) { t -= len; ++ti; --len; }
    tj = ti + t;
    if (!SYM) { const int x = ti; ti = tj; tj = x; }   // lower triangle: row tile >= column tile
  } else if (d.k_tri) {
    // longest sums (last column tiles) first
    tj = tiles_n - 1 - t / tiles_m;
    ti = t - (tiles_n - 1 - tj) * tiles_m;
  } else {
    ti = t / tiles_n;
    tj = t - ti * tiles_n;
  }
  const int m0 = ti * BTt, n0 = tj * BTt;
  const T* A = d.A + (long long)b * d.sA;
  const T* B = d.B + (long long)b * d.sB;
  const int Keff = d.k_tri && n0 + BTt < d.K ? n0 + BTt : d.K;

  acc_t acc[TI][TI];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TI; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

  // double buffered: the global loads of stage s+1 are in flight while stage s is multiplied
  const int KT_all = (Keff + BK - 1) / BK;
  const int per_split = (KT_all + (int)gridDim.y - 1) / (int)gridDim.y;
  const int kt0 = split * per_split;
  const int KT = KT_all - kt0 < per_split ? KT_all - kt0 : per_split;   // may be <= 0 for the last slices
  T pa[H][4], pb[H][4];
#define DA_RFETCH(kt)                                                                               \
  do {                                                                                              \
    _Pragma("unroll") for (int h = 0; h < H; ++h) {                                                 \
      fetch<A_KS>(pa[h], A, d.lda, m0 + 64 * h, (kt) * BK, d.M, Keff, tid);                         \
      fetch<B_KS>(pb[h], B, d.ldb, n0 + 64 * h, (kt) * BK, d.N, Keff, tid);                         \
    }                                                                                               \
  } while (0)
#define DA_RPUT(buf)                                                                                \
  do {                                                                                              \
    _Pragma("unroll") for (int h = 0; h < H; ++h) {                                                 \
      put<A_KS, BTt>(lds_a[buf] + 64 * h, pa[h], tid);                                              \
      put<B_KS, BTt>(lds_b[buf] + 64 * h, pb[h], tid);                                              \
    }                                                                                               \
  } while (0)
#define DA_RMMA(sa, sb)                                                                             \
  _Pragma("unroll") for (int ks = 0; ks < BK / 4; ++ks) {                                           \
    const int k = ks * 4 + (lane >> 4);                                                             \
    T af[TI], bfv[TI];                                                                              \
    _Pragma("unroll") for (int i = 0; i < TI; ++i) af[i] = (sa)[k * BTt + wm * WT + i * 16 + (lane & 15)];  \
    _Pragma("unroll") for (int j = 0; j < TI; ++j) bfv[j] = (sb)[k * BTt + wn * WT + j * 16 + (lane & 15)]; \
    _Pragma("unroll") for (int i = 0; i < TI; ++i)                                                  \
      _Pragma("unroll") for (int j = 0; j < TI; ++j) acc[i][j] = Mfma<T>::mma(af[i], bfv[j], acc[i][j]);    \
  }
  // Interior tile with 16-byte aligned operand rows: the stage loads need no range or alignment checks and
  // walk precomputed pointers.  (With the checks the loop issues ~380 scalar and vector ALU instructions per
  // stage around 16 MFMAs, more issue time than the MFMAs take.)
  const bool interior = m0 + BTt <= d.M && n0 + BTt <= d.N && Keff % BK == 0 &&
                        ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 &&
                        (((long long)d.lda | (long long)d.ldb) * (long long)sizeof(T)) % 16 == 0;
  if (interior) {
    // the thread's first element of each operand and the distance between stages
    const T* pA[H];
    const T* pB[H];
#pragma unroll
    for (int h = 0; h < H; ++h) {
      pA[h] = A_KS ? A + (long long)(kt0 * BK + (tid >> 4)) * d.lda + m0 + 64 * h + (tid & 15) * 4
                   : A + (long long)(m0 + 64 * h + (tid >> 2)) * d.lda + kt0 * BK + (tid & 3) * 4;
      pB[h] = B_KS ? B + (long long)(kt0 * BK + (tid >> 4)) * d.ldb + n0 + 64 * h + (tid & 15) * 4
                   : B + (long long)(n0 + 64 * h + (tid >> 2)) * d.ldb + kt0 * BK + (tid & 3) * 4;
    }
    const long long stepA = A_KS ? (long long)BK * d.lda : BK, stepB = B_KS ? (long long)BK * d.ldb : BK;
#define DA_RFETCH_FAST()                                                                            \
  do {                                                                                              \
    _Pragma("unroll") for (int h = 0; h < H; ++h) {                                                 \
      fetch_fast(pa[h], pA[h]);                                                                     \
      fetch_fast(pb[h], pB[h]);                                                                     \
      pA[h] += stepA;                                                                               \
      pB[h] += stepB;                                                                               \
    }                                                                                               \
  } while (0)
    if (KT > 0) {
      DA_RFETCH_FAST();
      DA_RPUT(0);
    }
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      const T* sa = lds_a[kt & 1];
      const T* sb = lds_b[kt & 1];
      const bool more = kt + 1 < KT;
      if (more) DA_RFETCH_FAST();
      DA_RMMA(sa, sb)
      if (more) DA_RPUT((kt + 1) & 1);
      __syncthreads();
    }
#undef DA_RFETCH_FAST
  } else {
    if (KT > 0) {
      DA_RFETCH(kt0);
      DA_RPUT(0);
    }
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      const T* sa = lds_a[kt & 1];
      const T* sb = lds_b[kt & 1];
      const bool more = kt + 1 < KT;
      if (more) DA_RFETCH(kt0 + kt + 1);
      DA_RMMA(sa, sb)
      if (more) DA_RPUT((kt + 1) & 1);
      __syncthreads();
    }
  }
#undef DA_RMMA
#undef DA_RFETCH
#undef DA_RPUT

  if (d.c_store != DA_STORE_NATIVE) {   // rounded once to the storage dtype; no E, no split, no mirror (checked on the host)
    char* Cc = reinterpret_cast<char*>(d.C) + (long long)b * d.sC * (d.c_store == DA_STORE_F32 ? 4 : 2);
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TI; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = m0 + wm * WT + i * 16 + Mfma<T>::row(v, lane);
          const int n = n0 + wn * WT + j * 16 + (lane & 15);
          if (m < d.M && n < d.N) {
            const float o = (float)((T)d.alpha * acc[i][j][v]);
            const long long at = (long long)m * d.ldc + n;
            if (d.c_store == DA_STORE_F32) reinterpret_cast<float*>(Cc)[at] = o;
            else reinterpret_cast<bf16_t*>(Cc)[at] = f2bf(o);
          }
        }
    return;
  }
  T* C = d.C + (long long)b * d.sC + (long long)split * d.split_stride;   // each K slice has an output of its own
  const T* E = d.E ? d.E + (long long)b * d.sE : nullptr;
  const bool mirror = SYM && (ti != tj);
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TI; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = m0 + wm * WT + i * 16 + Mfma<T>::row(v, lane);
        const int n = n0 + wn * WT + j * 16 + (lane & 15);
        if (m < d.M && n < d.N) {
          T o = (T)d.alpha * acc[i][j][v];
          if (E) o += (T)d.beta * E[(long long)m * d.lde + n];
          C[(long long)m * d.ldc + n] = o;
          if (mirror) C[(long long)n * d.ldc + m] = o;
        }
      }
}

template <typename T, int BTt>
long long blocks_of(const RealGemmDesc<T>& d) {
  const long long tiles_m = (d.M + BTt - 1) / BTt, tiles_n = (d.N + BTt - 1) / BTt;
  return ((d.symmetric || d.lower_only) ? tiles_n * tiles_m - tiles_n * (tiles_n - 1) / 2 : tiles_m * tiles_n) * d.batch;
}

template <typename T, bool A_KS, bool B_KS, bool SYM, int BTt>
int launch_bt(const RealGemmDesc<T>& d, int split, hipStream_t s) {
  const long long blocks = blocks_of<T, BTt>(d);
  if (blocks <= 0 || blocks > 0x7fffffffLL) return DA_ERR_LIMIT;
  hipLaunchKernelGGL((gemm_f64_kernel<T, A_KS, B_KS, SYM, BTt>), dim3((unsigned)blocks, split), dim3(256), 0, s, d);
  return da_launch_status();
}

template <typename T, bool A_KS, bool B_KS, bool SYM>
int launch(const RealGemmDesc<T>& d, hipStream_t s) {
  // Only the 64-wide tile is instantiated: the 128-wide one (half the operand bytes per flop, but 200 VGPRs
  // and 64 KB of LDS in fp64, i.e. two workgroups per CU instead of five) measured 10 % slower on the
  // orthonormaliser's large products and equal on the small ones.
  constexpr int BTt = 64;
  const long long blocks = blocks_of<T, BTt>(d);
  const bool auto_split = d.split_k < 0 && !d.E && d.c_store == DA_STORE_NATIVE;
  int split = d.split_k > 1 && !d.E ? d.split_k : 1;
  if (auto_split) split = da_auto_split(blocks, d.K);
  if (split > 1 && d.split_stride < (long long)d.sC * d.batch) return DA_ERR_ARG;
  return launch_bt<T, A_KS, B_KS, SYM, BTt>(d, split, s);
}

// Element-wise conversions of `batch` matrices of `per` contiguous elements; blockIdx.y = matrix.
__device__ __forceinline__ bool gate_open(const int* flags, int want, int b) {
  return !flags || (flags[b] != 0) == (want != 0);
}

template <typename T, typename R>
__global__ __launch_bounds__(256) void cvt_up_kernel(const T* __restrict__ src, R* __restrict__ dst, long long per,
                                                     const int* gate, int want) {
  const long long b = blockIdx.y;
  if (!gate_open(gate, want, (int)b)) return;
  src += b * per; dst += b * per;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < per; i += (long long)gridDim.x * 256)
    dst[i] = (R)ld_as_float<T>(src + i);
}

template <typename T, typename R>
__global__ __launch_bounds__(256) void cvt_down_kernel(const R* __restrict__ src, T* __restrict__ dst, long long per,
                                                       const int* gate, int want) {
  const long long b = blockIdx.y;
  if (!gate_open(gate, want, (int)b)) return;
  src += b * per; dst += b * per;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < per; i += (long long)gridDim.x * 256)
    st_from_float<T>(dst + i, (float)src[i]);
}

// R (fp64 / fp32) -> fp32 (unless dst is null) and, if `low` is given, the same values rounded once more to bf16
template <typename R>
__global__ __launch_bounds__(256) void cvt_f32_low_kernel(const R* __restrict__ src, float* __restrict__ dst,
                                                          bf16_t* __restrict__ low, long long per, const int* gate,
                                                          int want) {
  const long long b = blockIdx.y;
  if (!gate_open(gate, want, (int)b)) return;
  src += b * per;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < per; i += (long long)gridDim.x * 256) {
    const float v = (float)src[i];
    if (dst) dst[b * per + i] = v;
    if (low) low[b * per + i] = f2bf(v);
  }
}

// fp64 -> h + l (bf16 each): h = the value rounded to bf16, l = what is left of it, rounded to bf16
__global__ __launch_bounds__(256) void cvt_hl_kernel(const double* __restrict__ src, bf16_t* __restrict__ h,
                                                     bf16_t* __restrict__ l, long long per, const int* gate, int want) {
  const long long b = blockIdx.y;
  if (!gate_open(gate, want, (int)b)) return;
  src += b * per;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < per; i += (long long)gridDim.x * 256) {
    const float v = (float)src[i];
    const bf16_t hi = f2bf(v);
    h[b * per + i] = hi;
    l[b * per + i] = f2bf(v - bf2f(hi));
  }
}

inline dim3 cvt_grid(long long per, int batch) {
  long long b = (per + 255) / 256;
  const long long cap = 8192 / batch > 0 ? 8192 / batch : 1;
  if (b > cap) b = cap;
  return dim3((unsigned)(b < 1 ? 1 : b), (unsigned)batch);
}

template <typename T>
int gemm_real(const RealGemmDesc<T>& d, hipStream_t s) {
  if (!d.A || !d.B || !d.C || d.M <= 0 || d.N <= 0 || d.K < 0 || d.batch <= 0) return DA_ERR_ARG;
  if (d.lower_only && (d.M < d.N || d.symmetric)) return DA_ERR_ARG;
  if (d.c_store != DA_STORE_NATIVE && d.c_store != DA_STORE_BF16 && d.c_store != DA_STORE_F32) return DA_ERR_DTYPE;
  if (d.c_store != DA_STORE_NATIVE && (d.E || d.split_k > 1 || d.symmetric)) return DA_ERR_ARG;
  if (d.k_tri && (d.symmetric || d.lower_only || d.split_k > 1)) return DA_ERR_ARG;
  if (d.symmetric) {
    if (d.M != d.N || !d.a_kstrided || !d.b_kstrided) return DA_ERR_ARG;  // only the Gram form A^T A
    return launch<T, true, true, true>(d, s);
  }
  if (!d.a_kstrided && !d.b_kstrided) return launch<T, false, false, false>(d, s);
  if (!d.a_kstrided && d.b_kstrided) return launch<T, false, true, false>(d, s);
  if (d.a_kstrided && !d.b_kstrided) return launch<T, true, false, false>(d, s);
  return launch<T, true, true, false>(d, s);
}

template <typename R>
int cvt_up(const void* src, int src_dtype, R* dst, long long per, int batch, DaGate g, hipStream_t s) {
  if (per <= 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  if (src_dtype == DA_BF16)
    hipLaunchKernelGGL((cvt_up_kernel<bf16_t, R>), cvt_grid(per, batch), dim3(256), 0, s, static_cast<const bf16_t*>(src), dst, per, g.flags, g.want);
  else if (src_dtype == DA_F32)
    hipLaunchKernelGGL((cvt_up_kernel<float, R>), cvt_grid(per, batch), dim3(256), 0, s, static_cast<const float*>(src), dst, per, g.flags, g.want);
  else
    return DA_ERR_DTYPE;
  return da_launch_status();
}

}  // namespace

int da_gemm_f64(const Gemm64Desc& d, hipStream_t s) { return gemm_real<double>(d, s); }
int da_gemm_f32s(const Gemm32Desc& d, hipStream_t s) { return gemm_real<float>(d, s); }

int da_cvt_to_f64(const void* src, int src_dtype, double* dst, long long per, int batch, DaGate g, hipStream_t s) {
  return cvt_up<double>(src, src_dtype, dst, per, batch, g, s);
}
int da_cvt_to_f32(const void* src, int src_dtype, float* dst, long long per, int batch, DaGate g, hipStream_t s) {
  return cvt_up<float>(src, src_dtype, dst, per, batch, g, s);
}
int da_cvt_from_f64(const double* src, void* dst, int dst_dtype, long long per, int batch, DaGate g, hipStream_t s) {
  if (per <= 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  if (dst_dtype == DA_BF16)
    hipLaunchKernelGGL((cvt_down_kernel<bf16_t, double>), cvt_grid(per, batch), dim3(256), 0, s, src, static_cast<bf16_t*>(dst), per, g.flags, g.want);
  else if (dst_dtype == DA_F32)
    hipLaunchKernelGGL((cvt_down_kernel<float, double>), cvt_grid(per, batch), dim3(256), 0, s, src, static_cast<float*>(dst), per, g.flags, g.want);
  else
    return DA_ERR_DTYPE;
  return da_launch_status();
}
int da_cvt_from_f32(const float* src, void* dst, int dst_dtype, long long per, int batch, DaGate g, hipStream_t s) {
  if (per <= 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  if (dst_dtype == DA_BF16)
    hipLaunchKernelGGL((cvt_down_kernel<bf16_t, float>), cvt_grid(per, batch), dim3(256), 0, s, src, static_cast<bf16_t*>(dst), per, g.flags, g.want);
  else if (dst_dtype == DA_F32)
    hipLaunchKernelGGL((cvt_down_kernel<float, float>), cvt_grid(per, batch), dim3(256), 0, s, src, static_cast<float*>(dst), per, g.flags, g.want);
  else
    return DA_ERR_DTYPE;
  return da_launch_status();
}
int da_cvt_f64_to_hl(const double* src, bf16_t* h, bf16_t* l, long long per, int batch, DaGate g, hipStream_t s) {
  if (per <= 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  hipLaunchKernelGGL(cvt_hl_kernel, cvt_grid(per, batch), dim3(256), 0, s, src, h, l, per, g.flags, g.want);
  return da_launch_status();
}
int da_cvt_f64_to_f32(const double* src, float* dst, bf16_t* low, long long per, int batch, DaGate g, hipStream_t s) {
  if (per <= 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  hipLaunchKernelGGL(cvt_f32_low_kernel<double>, cvt_grid(per, batch), dim3(256), 0, s, src, dst, low, per, g.flags, g.want);
  return da_launch_status();
}
int da_cvt_f32_to_bf16(const float* src, bf16_t* low, long long per, int batch, DaGate g, hipStream_t s) {
  if (per <= 0 || batch <= 0 || batch > 65535) return DA_ERR_ARG;
  hipLaunchKernelGGL(cvt_f32_low_kernel<float>, cvt_grid(per, batch), dim3(256), 0, s, src, static_cast<float*>(nullptr), low, per, g.flags, g.want);
  return da_launch_status();
}
