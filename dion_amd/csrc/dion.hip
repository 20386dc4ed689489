// Dion step building blocks that are not GEMMs: the momentum accumulation with its all-zero
// guard, dtype casts, the NaN / all-zero fix-up of P and R, the column normalisation that
// turns R into the next Q, and the host-side driver of the orthonormalisation (one blocked
// CholeskyQR pass in fp64: Gram -> Cholesky -> triangular solve, then closed-form polishing passes).
#include "dion.h"
#include "gemm_f64.h"
#include "prof.h"

namespace {

template <typename T> struct V8;
template <> struct V8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = bf2f((bf16_t)(w[i] & 0xffffu));
      v[2 * i + 1] = bf2f((bf16_t)(w[i] >> 16));
    }
  }
  // read-once data (gradients): keep it out of the caches' way
  static __device__ __forceinline__ void load_nt(const bf16_t* p, float (&v)[8]) {
    typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
    const u32x4_t r = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned w = r[i];
      v[2 * i] = bf2f((bf16_t)(w & 0xffffu));
      v[2 * i + 1] = bf2f((bf16_t)(w >> 16));
    }
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f2bf(v[2 * i]) | ((uint32_t)f2bf(v[2 * i + 1]) << 16);
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  static __device__ __forceinline__ float round(float x) { return rbf(x); }
  static __device__ __forceinline__ float maxval() { return 3.3895313892515355e38f; }
};
template <> struct V8<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void load_nt(const float* p, float (&v)[8]) {
    typedef float f32x4_nt_t __attribute__((ext_vector_type(4)));
    const f32x4_nt_t a = __builtin_nontemporal_load(reinterpret_cast<const f32x4_nt_t*>(p));
    const f32x4_nt_t b = __builtin_nontemporal_load(reinterpret_cast<const f32x4_nt_t*>(p + 4));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float x = a[i], y = b[i];
      v[i] = x; v[4 + i] = y;
    }
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
  static __device__ __forceinline__ float round(float x) { return x; }
  static __device__ __forceinline__ float maxval() { return 3.4028234663852886e38f; }
};

__global__ void fill_int_kernel(int* p, int n, int v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// Start of a bucket chunk in one launch: the two device pointer tables and the cleared per-matrix words.
__global__ void dion_setup_kernel(DaPtrTable ta, void** dst_a, DaPtrTable tb, void** dst_b, int n, int* nonzero,
                                  int* info) {
  const int i = threadIdx.x;
  if (i < n) {
    dst_a[i] = ta.p[i];
    dst_b[i] = tb.p[i];
    nonzero[i] = 0;
    info[i] = 0;
  }
}

// M <- M + G (rounded to M's dtype); nonzero[b] |= any(M != 0).
template <typename TM, typename TG>
__global__ __launch_bounds__(256) void add_grad_kernel(DaPtrTable mt, DaPtrTable gt, long long n, int* nonzero) {
  const int b = blockIdx.y;
  TM* M = static_cast<TM*>(mt.p[b]);
  const TG* G = static_cast<const TG*>(gt.p[b]);
  bool any = false;
  for (long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long long)gridDim.x * 256 * 8) {
    float m[8], g[8];
    V8<TM>::load(M + i, m);
    V8<TG>::load_nt(G + i, g);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      m[e] = V8<TM>::round(m[e] + g[e]);
      any |= (m[e] != 0.f);
    }
    V8<TM>::store(M + i, m);
  }
  // every writer stores the same value: no atomic needed
  if (__any(any) && (threadIdx.x & 63) == 0) nonzero[b] = 1;
}

// dst[b] (contiguous, TD) <- src table[b] (TS)
template <typename TS, typename TD>
__global__ __launch_bounds__(256) void cast_table_kernel(DaPtrTable st, TD* dst, long long n) {
  const int b = blockIdx.y;
  const TS* S = static_cast<const TS*>(st.p[b]);
  TD* D = dst + (long long)b * n;
  for (long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long long)gridDim.x * 256 * 8) {
    float v[8];
    V8<TS>::load(S + i, v);
    V8<TD>::store(D + i, v);
  }
}

// dst[b] (rows x ld, contiguous, TD) <- src table[b] (rows x cols contiguous, TS); columns cols .. ld-1 are
// zeroed.  For a column count that is not a multiple of 8: the working copy gets 16-byte rows.
template <typename TS, typename TD>
__global__ __launch_bounds__(256) void cast_table_pitched_kernel(DaPtrTable st, TD* dst, int rows, int cols, int ld) {
  const int b = blockIdx.y;
  const TS* S = static_cast<const TS*>(st.p[b]);
  const long long n = (long long)rows * ld;
  TD* D = dst + (long long)b * n;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const long long row = i / ld;
    const int c = (int)(i - row * ld);
    st_from_float<TD>(D + i, c < cols ? ld_as_float<TS>(S + row * cols + c) : 0.f);
  }
}

// v <- nan_to_num(v) * nonzero + alt * (1 - nonzero)      (alt may be null: treated as 0)
template <typename T>
__global__ __launch_bounds__(256) void fix_kernel(T* V, const T* alt, long long n, const int* nonzero) {
  const int b = blockIdx.y;
  const bool nz = nonzero[b] != 0;
  T* p = V + (long long)b * n;
  const T* a = alt ? alt + (long long)b * n : nullptr;
  for (long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long long)gridDim.x * 256 * 8) {
    float v[8], q[8];
    V8<T>::load(p + i, v);
    if (a && !nz) V8<T>::load(a + i, q);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = v[e];
      if (x != x) x = 0.f;
      else if (x > V8<T>::maxval()) x = V8<T>::maxval();
      else if (x < -V8<T>::maxval()) x = -V8<T>::maxval();
      v[e] = nz ? x : (a ? q[e] : 0.f);
    }
    V8<T>::store(p + i, v);
  }
}

// The same fix-up for a product that was computed as `parts` partial sums over slices of its inner dimension
// (fp32, `pstride` elements apart): v <- round(sum of the parts), then as fix_kernel.
template <typename T>
__global__ __launch_bounds__(256) void fix_sum_kernel(const float* __restrict__ part, int parts, long long pstride,
                                                      T* V, const T* alt, long long n, const int* nonzero) {
  const int b = blockIdx.y;
  const bool nz = nonzero[b] != 0;
  T* p = V + (long long)b * n;
  const float* s0 = part + (long long)b * n;
  const T* a = alt ? alt + (long long)b * n : nullptr;
  for (long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long long)gridDim.x * 256 * 8) {
    float v[8], q[8];
    V8<float>::load(s0 + i, v);
    for (int k = 1; k < parts; ++k) {
      float t[8];
      V8<float>::load(s0 + k * pstride + i, t);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] += t[e];
    }
    if (a && !nz) V8<T>::load(a + i, q);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = V8<T>::round(v[e]);
      if (x != x) x = 0.f;
      else if (x > V8<T>::maxval()) x = V8<T>::maxval();
      else if (x < -V8<T>::maxval()) x = -V8<T>::maxval();
      v[e] = nz ? x : (a ? q[e] : 0.f);
    }
    V8<T>::store(p + i, v);
  }
}

// Column normalisation of R[b] (rows x r, TM): Qn = R / (sqrt(sum_rows R^2) + eps), computed in
// fp32 (column sums accumulated in fp64), stored as TM into qn[b] and, cast to TQ, into the
// optimizer's Q state (its first q_cols columns: the working matrices may carry zero columns up to a
// multiple of 8).  Three launches: partial column sums over row slices, their sum in slice order (so the
// result does not depend on which workgroup finishes first), then a fully parallel normalise pass.
template <typename TM>
__global__ __launch_bounds__(256) void colsum_kernel(const TM* __restrict__ R, double* __restrict__ part, int rows, int r,
                                                     int rows_per_slice) {
  __shared__ double red[4][64];
  const int b = blockIdx.z;
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  const int g = threadIdx.x >> 6;
  const TM* Rb = R + (long long)b * rows * r;
  const int i0 = blockIdx.y * rows_per_slice;
  const int i1 = i0 + rows_per_slice < rows ? i0 + rows_per_slice : rows;
  double s = 0.0;
  if (c < r)
    for (int i = i0 + g; i < i1; i += 4) {
      const float v = ld_as_float<TM>(Rb + (long long)i * r + c);
      s += (double)v * (double)v;
    }
  red[g][threadIdx.x & 63] = s;
  __syncthreads();
  if (g == 0 && c < r) {
    const double t = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
    part[((long long)blockIdx.y * gridDim.z + b) * r + c] = t;
  }
}

// sums[b][c] = part[0][b][c] + part[1][b][c] + ... in that order
__global__ __launch_bounds__(256) void colsum_finish_kernel(const double* __restrict__ part, double* __restrict__ sums,
                                                            int slices, long long per_slice) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= per_slice) return;
  double s = 0.0;
  for (int k = 0; k < slices; ++k) s += part[k * per_slice + i];
  sums[i] = s;
}

template <typename TM, typename TQ>
__global__ __launch_bounds__(256) void colscale_kernel(const TM* __restrict__ R, TM* __restrict__ qn, DaPtrTable qt,
                                                       const double* __restrict__ sums, long long n, int r, int q_cols,
                                                       float eps) {
  const int b = blockIdx.y;
  const TM* Rb = R + (long long)b * n;
  TM* Qn = qn + (long long)b * n;
  TQ* Q = static_cast<TQ*>(qt.p[b]);
  const double* sb = sums + (long long)b * r;
  for (long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long long)gridDim.x * 256 * 8) {
    const int c0 = (int)(i % r);  // r is a multiple of 8: the 8 elements stay in one row
    float v[8], q[8];
    V8<TM>::load(Rb + i, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float d = sqrtf((float)sb[c0 + e]) + eps;
      v[e] = V8<TM>::round(v[e] / d);     // cast back to R's dtype (reference dion/dion.py:1490)
      q[e] = v[e];
    }
    V8<TM>::store(Qn + i, v);
    // Q <- Q_new.to(Q.dtype) (reference dion/dion.py:1559-1561); the state has q_cols <= r columns, contiguous
    if (q_cols == r) {
      V8<TQ>::store(Q + i, q);
    } else {
      const long long row = i / r;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (c0 + e < q_cols) st_from_float<TQ>(Q + row * q_cols + c0 + e, q[e]);
    }
  }
}

inline unsigned ew_blocks(long long n) {
  long long b = (n / 8 + 255) / 256;
  return (unsigned)(b > 1024 ? 1024 : (b < 1 ? 1 : b));
}

}  // namespace

int da_fill_int(int* p, int n, int v, hipStream_t s) {
  hipLaunchKernelGGL(fill_int_kernel, dim3((n + 255) / 256), dim3(256), 0, s, p, n, v);
  return da_launch_status();
}

int da_dion_setup(const DaPtrTable& ta, void** dst_a, const DaPtrTable& tb, void** dst_b, int n, int* nonzero,
                  int* info, hipStream_t s) {
  if (n < 1 || n > DA_MAX_PTRS) return DA_ERR_LIMIT;
  hipLaunchKernelGGL(dion_setup_kernel, dim3(1), dim3(64), 0, s, ta, dst_a, tb, dst_b, n, nonzero, info);
  return da_launch_status();
}

int da_add_grad(const DaPtrTable& m, const DaPtrTable& g, int m_dtype, int g_dtype, long long n, int batch,
                int* nonzero, hipStream_t s) {
  if (n & 7) return DA_ERR_ALIGN;
  dim3 grid(ew_blocks(n), batch);
  if (m_dtype == DA_BF16 && g_dtype == DA_BF16)
    hipLaunchKernelGGL((add_grad_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, s, m, g, n, nonzero);
  else if (m_dtype == DA_BF16 && g_dtype == DA_F32)
    hipLaunchKernelGGL((add_grad_kernel<bf16_t, float>), grid, dim3(256), 0, s, m, g, n, nonzero);
  else if (m_dtype == DA_F32 && g_dtype == DA_BF16)
    hipLaunchKernelGGL((add_grad_kernel<float, bf16_t>), grid, dim3(256), 0, s, m, g, n, nonzero);
  else if (m_dtype == DA_F32 && g_dtype == DA_F32)
    hipLaunchKernelGGL((add_grad_kernel<float, float>), grid, dim3(256), 0, s, m, g, n, nonzero);
  else
    return DA_ERR_DTYPE;
  return da_launch_status();
}

int da_cast_table(const DaPtrTable& src, int s_dtype, void* dst, int d_dtype, int rows, int cols, int ld, int batch,
                  hipStream_t s) {
  if (rows <= 0 || cols <= 0 || ld < cols || (ld & 7)) return DA_ERR_ALIGN;
  const long long n = (long long)rows * ld;
  const bool flat = cols == ld;
  dim3 grid(flat ? ew_blocks(n) : ew_blocks(8 * n), batch);
#define DA_CAST_CASE(TS, TD)                                                                                      \
  do {                                                                                                            \
    if (flat)                                                                                                     \
      hipLaunchKernelGGL((cast_table_kernel<TS, TD>), grid, dim3(256), 0, s, src, static_cast<TD*>(dst), n);      \
    else                                                                                                          \
      hipLaunchKernelGGL((cast_table_pitched_kernel<TS, TD>), grid, dim3(256), 0, s, src, static_cast<TD*>(dst),  \
                         rows, cols, ld);                                                                         \
  } while (0)
  if (s_dtype == DA_BF16 && d_dtype == DA_BF16) DA_CAST_CASE(bf16_t, bf16_t);
  else if (s_dtype == DA_F32 && d_dtype == DA_BF16) DA_CAST_CASE(float, bf16_t);
  else if (s_dtype == DA_BF16 && d_dtype == DA_F32) DA_CAST_CASE(bf16_t, float);
  else if (s_dtype == DA_F32 && d_dtype == DA_F32) DA_CAST_CASE(float, float);
  else return DA_ERR_DTYPE;
#undef DA_CAST_CASE
  return da_launch_status();
}

int da_fix(void* v, const void* alt, int dtype, long long n, int batch, const int* nonzero, hipStream_t s) {
  if (n & 7) return DA_ERR_ALIGN;
  dim3 grid(ew_blocks(n), batch);
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(fix_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<bf16_t*>(v), static_cast<const bf16_t*>(alt), n, nonzero);
  else if (dtype == DA_F32)
    hipLaunchKernelGGL(fix_kernel<float>, grid, dim3(256), 0, s, static_cast<float*>(v), static_cast<const float*>(alt), n, nonzero);
  else
    return DA_ERR_DTYPE;
  return da_launch_status();
}

int da_fix_sum(const float* part, int parts, long long pstride, void* v, const void* alt, int dtype, long long n,
               int batch, const int* nonzero, hipStream_t s) {
  if ((n & 7) || (pstride & 7) || parts < 1) return DA_ERR_ALIGN;
  dim3 grid(ew_blocks(n), batch);
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(fix_sum_kernel<bf16_t>, grid, dim3(256), 0, s, part, parts, pstride, static_cast<bf16_t*>(v), static_cast<const bf16_t*>(alt), n, nonzero);
  else if (dtype == DA_F32)
    hipLaunchKernelGGL(fix_sum_kernel<float>, grid, dim3(256), 0, s, part, parts, pstride, static_cast<float*>(v), static_cast<const float*>(alt), n, nonzero);
  else
    return DA_ERR_DTYPE;
  return da_launch_status();
}

int da_colnorm(const void* R, void* qn, int m_dtype, const DaPtrTable& q, int q_dtype, int rows, int r, int q_cols,
               float eps, int batch, double* sums, hipStream_t s) {
  if ((r & 7) || q_cols < 1 || q_cols > r) return DA_ERR_ALIGN;
  const long long ns = (long long)batch * r;
  // 64 rows per workgroup (16 per row group): enough workgroups to pull R at the memory system's rate
  int slices = (rows + 63) / 64;
  if (slices > 1024) slices = 1024;
  const int rps = (rows + slices - 1) / slices;
  double* part = sums + ns;   // [slices][batch][r]
  dim3 g1((r + 63) / 64, slices, batch);
  if (m_dtype == DA_BF16)
    hipLaunchKernelGGL(colsum_kernel<bf16_t>, g1, dim3(256), 0, s, static_cast<const bf16_t*>(R), part, rows, r, rps);
  else if (m_dtype == DA_F32)
    hipLaunchKernelGGL(colsum_kernel<float>, g1, dim3(256), 0, s, static_cast<const float*>(R), part, rows, r, rps);
  else
    return DA_ERR_DTYPE;
  hipLaunchKernelGGL(colsum_finish_kernel, dim3((unsigned)((ns + 255) / 256)), dim3(256), 0, s, part, sums, slices, ns);
  const long long n = (long long)rows * r;
  dim3 g2(ew_blocks(n), batch);
  if (m_dtype == DA_BF16 && q_dtype == DA_BF16)
    hipLaunchKernelGGL((colscale_kernel<bf16_t, bf16_t>), g2, dim3(256), 0, s, static_cast<const bf16_t*>(R), static_cast<bf16_t*>(qn), q, sums, n, r, q_cols, eps);
  else if (m_dtype == DA_BF16 && q_dtype == DA_F32)
    hipLaunchKernelGGL((colscale_kernel<bf16_t, float>), g2, dim3(256), 0, s, static_cast<const bf16_t*>(R), static_cast<bf16_t*>(qn), q, sums, n, r, q_cols, eps);
  else if (m_dtype == DA_F32 && q_dtype == DA_BF16)
    hipLaunchKernelGGL((colscale_kernel<float, bf16_t>), g2, dim3(256), 0, s, static_cast<const float*>(R), static_cast<float*>(qn), q, sums, n, r, q_cols, eps);
  else if (m_dtype == DA_F32 && q_dtype == DA_F32)
    hipLaunchKernelGGL((colscale_kernel<float, float>), g2, dim3(256), 0, s, static_cast<const float*>(R), static_cast<float*>(qn), q, sums, n, r, q_cols, eps);
  else
    return DA_ERR_DTYPE;
  return da_launch_status();
}

// ---------------------------------------------------------------------------------------
// CholeskyQR2 in fp64
// ---------------------------------------------------------------------------------------
size_t da_orth_workspace_bytes(int batch, int rows, int r) {
  size_t per = (size_t)rows * r * 8       // P in fp64, orthonormalised in place (first pass)
               + 3 * (size_t)r * r * 8    // G, L, W (fp64; the polishing passes keep their fp32 G and V there)
               + (size_t)rows * r * 4     // the fp64 pass's result in fp32 (input of the polishing pass)
               + (size_t)rows * r * 2;    // ... and in bf16 (operand of its correction product)
  return per * batch + 256;
}

namespace {

// G[b][i][i] = 1 for r_live <= i < r: the Gram matrix of a P whose last r - r_live columns are zero becomes
// block diagonal with an identity block, and the factorisation leaves those columns of P zero.
__global__ void pad_diag_kernel(double* G, long long rr, int r, int r_live) {
  const int i = r_live + threadIdx.x;
  if (i < r) G[blockIdx.x * rr + (long long)i * r + i] = 1.0;
}

// One blocked CholeskyQR pass in fp64, in place:  P <- P R^-1  with  P^T P = R^T R.
int cholqr_pass(double* P0, double* G, double* L, double* W, int batch, int rows, int r, int r_live, bool g_cleared,
                int* info, hipStream_t s) {
  const int NB = DA_CHOL_NB;
  const int nblk = (r + NB - 1) / NB;
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  Gemm64Desc g{};
  g.batch = batch;
  // G = P0^T P0
  g.A = P0; g.B = P0; g.C = G; g.E = nullptr;
  g.sA = pr; g.sB = pr; g.sC = rr;
  g.lda = r; g.ldb = r; g.ldc = r;
  g.M = r; g.N = r; g.K = rows;
  g.a_kstrided = 1; g.b_kstrided = 1; g.symmetric = 1; g.alpha = 1.0; g.beta = 0.0;
  g.split_k = -1;   // few output tiles, long K: the launcher slices K until the GPU is full
  g.c_is_zero = g_cleared ? 1 : 0;
  int rc = da_gemm_f64(g, s);
  if (rc) return rc;
  if (r_live < r) {
    hipLaunchKernelGGL(pad_diag_kernel, dim3((unsigned)batch), dim3(64), 0, s, G, rr, r, r_live);
    rc = da_launch_status();
    if (rc) return rc;
  }
  // blocked lower Cholesky G = L L^T (right-looking), building W alongside
  for (int j = 0; j < nblk; ++j) {
    const int o = j * NB, nb = r - o < NB ? r - o : NB, rest = r - o - nb;
    rc = da_chol_step(G, L, W, rr, r, o, nb, info, batch, s);
    if (rc) return rc;
    if (rest <= 0) break;
    // A22 -= L21 L21^T, lower triangle only (nothing reads the upper one)
    Gemm64Desc u{};
    u.batch = batch;
    u.A = L + (long long)(o + nb) * r + o; u.sA = rr; u.lda = r; u.a_kstrided = 0;
    u.B = u.A; u.sB = rr; u.ldb = r; u.b_kstrided = 0;
    u.C = G + (long long)(o + nb) * r + (o + nb); u.sC = rr; u.ldc = r;
    u.E = u.C; u.sE = rr; u.lde = r;
    u.M = rest; u.N = rest; u.K = nb; u.alpha = -1.0; u.beta = 1.0; u.lower_only = 1;
    rc = da_gemm_f64(u, s);
    if (rc) return rc;
  }
  // P0 <- P0 R^-1 with R = L^T, in place, block column by block column:
  //   P0[:, j] <- P0[:, 0 .. j] W[j, 0 .. j]^T
  // (each workgroup owns 64 rows and the one 64-column output tile, and has read all it needs of
  // those rows before it stores)
  for (int j = 0; j < nblk; ++j) {
    const int o = j * NB, nb = r - o < NB ? r - o : NB;
    Gemm64Desc a{};
    a.batch = batch;
    a.A = P0; a.sA = pr; a.lda = r; a.a_kstrided = 0;
    a.B = W + (long long)o * r; a.sB = rr; a.ldb = r; a.b_kstrided = 0;
    a.C = P0 + o; a.sC = pr; a.ldc = r;
    a.E = nullptr;
    a.M = rows; a.N = nb; a.K = o + nb; a.alpha = 1.0; a.beta = 0.0;
    rc = da_gemm_f64(a, s);
    if (rc) return rc;
  }
  return DA_OK;
}

// V = I - up(G - I) for each r x r Gram matrix G of an almost orthonormal P, where up() keeps the strict
// upper triangle and half of the diagonal: the Cholesky factor of G = I + E is R = I + up(E) + O(E^2), so
// P V = P R^-1 + O(E^2).
__global__ __launch_bounds__(256) void polish_factor_kernel(const float* __restrict__ G, float* __restrict__ V,
                                                            long long rr, int r) {
  const long long b = blockIdx.y;
  const int i = blockIdx.x;
  const float* g = G + b * rr + (long long)i * r;
  float* v = V + b * rr + (long long)i * r;
  for (int j = threadIdx.x; j < r; j += 256) {
    const float x = g[j];
    v[j] = i < j ? -x : (i == j ? 1.5f - 0.5f * x : 0.f);
  }
}

// U = up(G - I) in bf16 (see polish_factor_kernel): the factor of the correction product P U, which only has
// to be known to the relative accuracy of bf16 because it is itself of the size of the defect.
__global__ __launch_bounds__(256) void polish_correction_kernel(const float* __restrict__ G, bf16_t* __restrict__ U,
                                                                long long rr, int r) {
  const long long b = blockIdx.y;
  const int i = blockIdx.x;
  const float* g = G + b * rr + (long long)i * r;
  bf16_t* u = U + b * rr + (long long)i * r;
  for (int j = threadIdx.x; j < r; j += 256) {
    const float x = g[j];
    u[j] = f2bf(i < j ? x : (i == j ? 0.5f * (x - 1.f) : 0.f));
  }
}

// The last polishing pass of an iterate that exists in fp32 and in bf16:  out <- in - in_bf16 U(in^T in).
// The Gram product is fp32 as in polish_pass; the correction product runs on the bf16 matrix cores (its
// relative error 2^-8 times the defect E of `in` adds 4e-3 E to the result, next to the pass's own O(E^2)).
int polish_pass_bf16(const float* in, const bf16_t* in_low, void* out, int out_dtype, float* G, bf16_t* U, int batch,
                     int rows, int r, bool g_cleared, hipStream_t s) {
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  Gemm32Desc g{};
  g.batch = batch;
  g.A = in; g.B = in; g.C = G;
  g.sA = pr; g.sB = pr; g.sC = rr;
  g.lda = r; g.ldb = r; g.ldc = r;
  g.M = r; g.N = r; g.K = rows;
  g.a_kstrided = 1; g.b_kstrided = 1; g.symmetric = 1; g.alpha = 1.0; g.beta = 0.0;
  g.split_k = -1;
  g.c_is_zero = g_cleared ? 1 : 0;
  int rc = da_gemm_f32s(g, s);
  if (rc) return rc;
  hipLaunchKernelGGL(polish_correction_kernel, dim3((unsigned)r, (unsigned)batch), dim3(256), 0, s, G, U, rr, r);
  rc = da_launch_status();
  if (rc) return rc;
  GemmDesc c{};
  c.batch = batch;
  c.A = in_low; c.sA = pr; c.lda = r; c.a_kstrided = 0;
  c.B = U; c.sB = rr; c.ldb = r; c.b_kstrided = 1;
  c.C = out; c.sC = pr; c.ldc = r; c.c_dtype = out_dtype;
  // the addend has C's dtype: the fp32 iterate for an fp32 result, its bf16 copy for a bf16 one
  c.E = out_dtype == DA_F32 ? static_cast<const void*>(in) : static_cast<const void*>(in_low);
  c.sE = pr; c.lde = r;
  c.M = rows; c.N = r; c.K = r;
  c.epilogue = DA_EPI_AXPBY; c.s0 = 1.f; c.s1 = -1.f; c.faithful = 0;
  return da_gemm_bf16(c, s);
}

// One polishing pass in fp32:  out <- in V(in^T in).  `in` (fp32) and `out` (fp32, or the caller's dtype for
// the last pass) are different buffers; one Gram product, one elementwise pass over r x r, one product with
// the triangular V -- no serial chain.
int polish_pass(const float* in, void* out, int out_store, float* G, float* V, int batch, int rows, int r,
                bool g_cleared, hipStream_t s) {
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  Gemm32Desc g{};
  g.batch = batch;
  g.A = in; g.B = in; g.C = G;
  g.sA = pr; g.sB = pr; g.sC = rr;
  g.lda = r; g.ldb = r; g.ldc = r;
  g.M = r; g.N = r; g.K = rows;
  g.a_kstrided = 1; g.b_kstrided = 1; g.symmetric = 1; g.alpha = 1.0; g.beta = 0.0;
  g.split_k = -1;
  g.c_is_zero = g_cleared ? 1 : 0;
  int rc = da_gemm_f32s(g, s);
  if (rc) return rc;
  hipLaunchKernelGGL(polish_factor_kernel, dim3((unsigned)r, (unsigned)batch), dim3(256), 0, s, G, V, rr, r);
  rc = da_launch_status();
  if (rc) return rc;
  // out = in V: V is upper triangular, so column tile j only sums k < 64 (j + 1)
  Gemm32Desc a{};
  a.batch = batch;
  a.A = in; a.sA = pr; a.lda = r; a.a_kstrided = 0;
  a.B = V; a.sB = rr; a.ldb = r; a.b_kstrided = 1;
  a.C = static_cast<float*>(out); a.c_store = out_store; a.sC = pr; a.ldc = r;
  a.M = rows; a.N = r; a.K = r; a.alpha = 1.0; a.beta = 0.0; a.k_tri = 1;
  return da_gemm_f32s(a, s);
}

}  // namespace

// The first pass is a blocked CholeskyQR in fp64: the Gram matrix squares P's condition number (up to
// 4e12 on the optimizer's inputs).  Its result is orthonormal to E = eps64 * cond(P)^2 <= 1e-4, and for
// such a matrix the second CholeskyQR pass has a closed form to O(E^2) <= 1e-8 -- below fp32 round-off,
// which is all the output dtype (fp32 or bf16) can hold: R^-1 = I - up(P^T P - I).  So the later passes
// are two fp32 products and no factorisation at all; the last one stores the output dtype.
// Columns r_live .. r-1 of P, if any, must be zero on entry and are zero on return (a caller pads the
// rank to a multiple of 8 this way); the polishing passes multiply them by finite factors only.
int da_orthonormalize(const void* P, void* out, int dtype, int batch, int rows, int r, int r_live, int passes,
                      void* ws, int* info, hipStream_t s) {
  if (passes < 1 || batch > 65535 || r_live < 1 || r_live > r || r - r_live > 63) return DA_ERR_ARG;
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  double* P0 = static_cast<double*>(ws);
  double* G = P0 + pr * batch;
  double* L = G + rr * batch;
  double* W = L + rr * batch;
  float* P0f = reinterpret_cast<float*>(W + rr * batch);
  bf16_t* P0h = reinterpret_cast<bf16_t*>(P0f + pr * batch);
  // the Gram products are split over K when they have few tiles: their output is cleared by the conversion
  // launch that precedes them rather than by one of its own
  const bool split = da_auto_split(da_gram_blocks(r, batch), rows) > 1;
  int rc = da_cvt_to_f64(P, dtype, P0, pr * batch, split ? G : nullptr, rr * batch, s);
  if (rc) return rc;
  rc = cholqr_pass(P0, G, L, W, batch, rows, r, r_live, split, info, s);
  if (rc) return rc;
  if (passes == 1) return da_cvt_from_f64(P0, out, dtype, pr * batch, s);
  // one conversion pass to fp32 costs less than reading fp64 twice in the polishing products
  // (the bf16 product moves 16-byte chunks: r a multiple of 8, else the all-fp32 form below)
  const bool low = passes == 2 && (r & 7) == 0;
  // the fp32 Gram matrix of the first polishing pass goes where G was: cleared here for its split-K product
  rc = da_cvt_f64_to_f32(P0, P0f, low ? P0h : nullptr, pr * batch, split ? reinterpret_cast<float*>(G) : nullptr,
                         rr * batch, s);
  if (rc) return rc;
  if (low)
    return polish_pass_bf16(P0f, P0h, out, dtype, reinterpret_cast<float*>(G), reinterpret_cast<bf16_t*>(L), batch,
                            rows, r, split, s);
  const float* cur = P0f;
  float* Gf = reinterpret_cast<float*>(G);
  float* Vf = reinterpret_cast<float*>(L);
  for (int pass = 1; pass < passes; ++pass) {
    const bool last = pass + 1 == passes;
    // intermediate iterates alternate between the fp32 buffer and (as fp32) the no longer needed P0
    float* other = cur == P0f ? reinterpret_cast<float*>(P0) : P0f;
    rc = polish_pass(cur, last ? out : static_cast<void*>(other), last ? da_store_of(dtype) : DA_STORE_NATIVE, Gf, Vf,
                     batch, rows, r, split && pass == 1, s);
    if (rc) return rc;
    cur = other;
  }
  return DA_OK;
}
