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

// sums[b][c] = sum over the slices of part[k][b][c], in a fixed order: 64 columns per workgroup, the slices cut into
// four contiguous runs (one per wavefront, each added in slice order), the four run sums added in run order
__global__ __launch_bounds__(256) void colsum_finish_kernel(const double* __restrict__ part, double* __restrict__ sums,
                                                            int slices, long long per_slice) {
  __shared__ double run[4][64];
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
  const long long i = (long long)blockIdx.x * 64 + lane;
  const int per_run = (slices + 3) / 4;
  const int k0 = q * per_run, k1 = k0 + per_run < slices ? k0 + per_run : slices;
  double s = 0.0;
  if (i < per_slice)
    for (int k = k0; k < k1; ++k) s += part[k * per_slice + i];
  run[q][lane] = s;
  __syncthreads();
  if (q == 0 && i < per_slice) sums[i] = ((run[0][lane] + run[1][lane]) + run[2][lane]) + run[3][lane];
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
  hipLaunchKernelGGL(colsum_finish_kernel, dim3((unsigned)((ns + 63) / 64)), dim3(256), 0, s, part, sums, slices, ns);
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
// Orthonormalisation: CholeskyQR in fp32 with a measured defect, CholeskyQR in fp64 where that is not enough,
// closed-form polishing pass
// ---------------------------------------------------------------------------------------
namespace {

// Slices of K of the Gram products of `batch` rows x r matrices (1: unsliced).
int gram_slices(int batch, int rows, int r) { return da_auto_split(da_gram_blocks(r, batch), rows); }

// The same for the Gram products on the bf16 matrix cores (`kinds` products in the launch): slices until about 256
// tiles of 256 x 256 exist, but each slice is another fp32 slab for the finishing pass to read, so no more of them
// than keep the slabs (r x r each) small beside the operand (rows x r): rows / 4r; each at least 512 rows deep and a
// multiple of the stage depth.  `ks` receives the rows per slice.
int gram16_slices(int batch, int rows, int r, int kinds, int* ks) {
  const long long tiles = (long long)kinds * batch * ((r + 255) / 256) * ((r + 255) / 256);
  long long nsl = (256 + tiles - 1) / tiles;
  const int by_slab = rows / (4 * r) > 0 ? rows / (4 * r) : 1;
  if (nsl > by_slab) nsl = by_slab;
  const int by_rows = rows / 512 > 0 ? rows / 512 : 1;
  if (nsl > by_rows) nsl = by_rows;
  if (nsl > 64) nsl = 64;
  const int per = (int)(((rows + nsl - 1) / nsl + 63) / 64 * 64);
  if (ks) *ks = per;
  return (rows + per - 1) / per;
}

size_t orth_align(size_t x) { return (x + 255) & ~(size_t)255; }

// Workspace of one call, carved in this order.
struct OrthWs {
  double* P0;      // rows x r per matrix, fp64: the fp64 pass works in place here
  float* Pf;       // ... fp32: the fp32 pass works in place here; later the fp64 pass's result for its polishing pass
  bf16_t* Ph;      // ... bf16 copy of Pf (operand of the correction product)
  double* G;       // r x r per matrix (fp64, or fp32 in the same place): Gram matrix
  double* L;       // Cholesky factor; later the correction factor of the polishing pass
  double* W;       // inverse-factor blocks
  double* part;    // K-slice outputs of a sliced Gram product
  float* rowdef;   // r per matrix: squared defect of each row of the polishing pass's Gram matrix
  float* rowdef_part;   // ... as partial sums per 64-column block
  int* need;       // per matrix: 1 = the fp32 pass was not enough, the fp64 pass runs
  int* info32;     // per matrix: status of the fp32 factorisation
  int* bad;        // r per matrix: 1 = the column is not usable (noise-level pivot), it is zeroed
  double* pstat;   // 2 per matrix: smallest and largest pivot of the fp64 factorisation
  int* polish;     // per matrix: 1 = the fp64 pass's result goes through the polishing pass
  int* direct;     // per matrix: 1 = it is the result as it is
  size_t bytes;
  OrthWs(void* ws, int batch, int rows, int r) {
    const size_t pr = (size_t)rows * r * batch, rr = (size_t)r * r * batch;
    const int sp = gram_slices(batch, rows, r);
    char* p = static_cast<char*>(ws);
    auto take = [&](size_t n) { char* q = p; p += orth_align(n); return q; };
    P0 = reinterpret_cast<double*>(take(pr * 8));
    Pf = reinterpret_cast<float*>(take(pr * 4));
    Ph = reinterpret_cast<bf16_t*>(take(pr * 2));
    G = reinterpret_cast<double*>(take(rr * 8));
    L = reinterpret_cast<double*>(take(rr * 8));
    W = reinterpret_cast<double*>(take(rr * 8));
    // K-slice outputs: `sp` slices of the fp64 / fp32 Gram kernels, or two fp32 slabs per slice of the bf16 one
    const size_t slabs16 = (size_t)2 * gram16_slices(batch, rows, r, 1, nullptr);   // (one product has the most slices)
    const size_t part_a = rr * 8 * (sp > 2 ? sp : 2), part_b = rr * 4 * slabs16;
    part = reinterpret_cast<double*>(take(part_a > part_b ? part_a : part_b));
    rowdef = reinterpret_cast<float*>(take((size_t)r * batch * 4));
    rowdef_part = reinterpret_cast<float*>(take((size_t)((r + 63) / 64) * r * batch * 4));
    need = reinterpret_cast<int*>(take((size_t)batch * 4));
    info32 = reinterpret_cast<int*>(take((size_t)batch * 4));
    bad = reinterpret_cast<int*>(take((size_t)r * batch * 4));
    pstat = reinterpret_cast<double*>(take((size_t)batch * 16));
    polish = reinterpret_cast<int*>(take((size_t)batch * 4));
    direct = reinterpret_cast<int*>(take((size_t)batch * 4));
    bytes = (size_t)(p - static_cast<char*>(ws));
  }
};

}  // namespace

size_t da_orth_workspace_bytes(int batch, int rows, int r) { return OrthWs(nullptr, batch, rows, r).bytes + 256; }

namespace {

__device__ __forceinline__ bool orth_gate_open(const int* flags, int want, int b) {
  return !flags || (flags[b] != 0) == (want != 0);
}

// Row i of G[b] = sum of the K slices in slice order (sp > 1; else G already holds the product); rows
// r_live .. r-1 get a one on the diagonal: the Gram matrix of a P whose last r - r_live columns are zero becomes
// block diagonal with an identity block, and the factorisation leaves those columns of P zero.
// rowdef (if given): sum_j (G[i][j] - delta_ij)^2, the row's share of the squared defect ||G - I||_F^2.
template <typename T>
__global__ __launch_bounds__(256) void gram_finish_kernel(const T* __restrict__ part, int sp, long long slice_stride,
                                                          T* __restrict__ G, long long rr, int r, int r_live,
                                                          float* __restrict__ rowdef, const int* gate, int want) {
  const int b = blockIdx.y, i = blockIdx.x;
  if (!orth_gate_open(gate, want, b)) return;
  T* g = G + b * rr + (long long)i * r;
  float acc = 0.f;
  for (int j = threadIdx.x; j < r; j += 256) {
    T v;
    if (sp > 1) {
      v = T(0);
      for (int q = 0; q < sp; ++q) v += part[q * slice_stride + b * rr + (long long)i * r + j];
    } else {
      v = g[j];
    }
    if (i >= r_live && j == i) v = T(1);
    if (sp > 1 || (i >= r_live && j == i)) g[j] = v;
    const float e = (float)v - (i == j ? 1.f : 0.f);
    acc += e * e;
  }
  if (rowdef) {
    __shared__ float red[256];
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
      if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
      __syncthreads();
    }
    if (threadIdx.x == 0) rowdef[(long long)b * r + i] = red[0];
  }
}

// After the fp32 pass: need[b] = the fp32 factorisation failed or left a defect ||P^T P - I||_F above `tol`
// (then the closed-form polishing pass could not bring it to round-off, and the fp64 pass takes the matrix over).
__global__ __launch_bounds__(64) void decide_fast_kernel(const float* __restrict__ rowdef, const int* __restrict__ info32,
                                                         int* __restrict__ need, int r, float tol2) {
  const int b = blockIdx.x;
  if (threadIdx.x != 0) return;
  float s = 0.f;
  for (int i = 0; i < r; ++i) s += rowdef[(long long)b * r + i];   // fixed order
  need[b] = (info32[b] != 0 || !(s <= tol2)) ? 1 : 0;
}

// After the fp64 pass: a column whose row of P^T P - I is not small (or not finite) came from a pivot at round-off
// level -- a numerically rank-deficient P; it is dropped (zeroed) and reported like a failed pivot.
__global__ __launch_bounds__(256) void decide_cols_kernel(const float* __restrict__ rowdef, int* __restrict__ bad,
                                                          int* __restrict__ info, int r, const int* gate, int want) {
  const int b = blockIdx.x;
  if (!orth_gate_open(gate, want, b)) return;
  __shared__ int first;
  if (threadIdx.x == 0) first = 0x7fffffff;
  __syncthreads();
  for (int j = threadIdx.x; j < r; j += 256) {
    const float d = rowdef[(long long)b * r + j];
    const int is_bad = !(d <= 0.25f) ? 1 : 0;
    bad[(long long)b * r + j] = is_bad;
    if (is_bad) atomicMin(&first, j);
  }
  __syncthreads();
  if (threadIdx.x == 0 && first != 0x7fffffff && info[b] == 0) info[b] = first + 1;
}

// out[:, j] = 0 for the dropped columns.
template <typename T>
__global__ __launch_bounds__(256) void zero_cols_kernel(T* __restrict__ out, const int* __restrict__ bad, int rows, int r,
                                                        const int* __restrict__ info, const int* gate, int want) {
  const int b = blockIdx.y;
  if (!orth_gate_open(gate, want, b) || info[b] == 0) return;
  const int* bd = bad + (long long)b * r;
  T* o = out + (long long)b * rows * r;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < (long long)rows * r; e += (long long)gridDim.x * 256)
    if (bd[e % r]) st_from_float<T>(o + e, 0.f);
}

inline int gemm_real(const Gemm64Desc& d, hipStream_t s) { return da_gemm_f64(d, s); }
inline int gemm_real(const Gemm32Desc& d, hipStream_t s) { return da_gemm_f32s(d, s); }
inline int chol_step_real(double* G, double* L, double* W, long long sG, int r, int o, int nb, int* info, int batch,
                          DaGate g, hipStream_t s, int o_prev, int c_end, double* pstat) {
  return da_chol_step(G, L, W, sG, r, o, nb, info, batch, g, s, o_prev, c_end, pstat);
}
inline int chol_step_real(float* G, float* L, float* W, long long sG, int r, int o, int nb, int* info, int batch,
                          DaGate g, hipStream_t s, int o_prev, int c_end, float*) {
  return da_chol_step_f32(G, L, W, sG, r, o, nb, info, batch, g, s, o_prev, c_end);
}

// G = P^T P (K-sliced if that fills the GPU; the slices are added in a fixed order), padded diagonal, and
// optionally the rows' squared defects.
template <typename T>
int gram(const T* P, T* G, T* part, int batch, int rows, int r, int r_live, float* rowdef, DaGate gate, hipStream_t s,
         bool unsliced = false) {
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  // (as the fall-back of flagged matrices: unsliced, so that no finishing launch is needed)
  const int sp = gate.flags || unsliced ? 1 : gram_slices(batch, rows, r);
  RealGemmDesc<T> g{};
  g.batch = batch;
  g.A = P; g.B = P; g.C = sp > 1 ? part : G; g.E = nullptr;
  g.sA = pr; g.sB = pr; g.sC = rr;
  g.lda = r; g.ldb = r; g.ldc = r;
  g.M = r; g.N = r; g.K = rows;
  g.a_kstrided = 1; g.b_kstrided = 1; g.symmetric = 1; g.alpha = 1.0; g.beta = 0.0;
  g.split_k = sp; g.split_stride = rr * batch;
  g.gate = gate.flags; g.gate_want = gate.want;
  int rc = gemm_real(g, s);
  if (rc) return rc;
  if (sp > 1 || r_live < r || rowdef) {
    hipLaunchKernelGGL(gram_finish_kernel<T>, dim3((unsigned)r, (unsigned)batch), dim3(256), 0, s, part, sp, rr * batch,
                       G, rr, r, r_live, rowdef, gate.flags, gate.want);
    rc = da_launch_status();
  }
  return rc;
}

// Most 64 x 64 tiles (over the batch) a trailing update may have to ride along in the next step's launch.
const long long DA_CHOL_DEFER_TILES = [] { const char* e = getenv("DION_AMD_CHOL_DEFER_TILES"); const long long v = e ? atoll(e) : 0; return v > 0 ? v : 256; }();

// Panel width (in 64-column steps) of the two-level blocking of chol_factor / apply_rinv.
int chol_panel_steps(int nblk, bool fallback) {
  static const int pw_env = [] {
    const char* e = getenv("DION_AMD_CHOL_PANEL");
    const int v = e ? atoi(e) : 0;
    return v > 0 ? v : 4;
  }();
  // As the pass for flagged matrices only (gated), most launches find nothing to do and what counts is their number:
  // one level, every trailing update deferred into the next step's launch.
  return fallback ? nblk : pw_env;
}

// Blocked lower Cholesky G = L L^T of each r x r matrix (G is overwritten), with the inverse-factor blocks W that
// apply_rinv uses.
template <typename T>
int chol_factor(T* G, T* L, T* W, int batch, int r, int* info, DaGate gate, hipStream_t s, T* pstat = nullptr) {
  const int NB = DA_CHOL_NB;
  const int nblk = (r + NB - 1) / NB;
  const long long rr = (long long)r * r;
  int rc = DA_OK;
  // Two-level blocking: 64-column steps inside panels of `pw` steps.  A step's rank-64 update reaches only the
  // rest of its panel's columns; what lies right of the panel gets one rank-(64 pw) update when the panel is done
  // (the trailing matrix is then read and written once per panel instead of once per step).
  const bool fallback = gate.flags != nullptr;
  const int pw = chol_panel_steps(nblk, fallback);
  // (the rank-64 updates inside a panel ride along in the next step's launch instead of taking one of their own)
  static const bool defer = [] { const char* e = getenv("DION_AMD_CHOL_NO_DEFER"); return !(e && atoi(e)); }();
  bool pending = false;   // the previous step left its update to the next launch
  // blocked lower Cholesky G = L L^T, building W alongside
  for (int j = 0; j < nblk; ++j) {
    const int o = j * NB, nb = r - o < NB ? r - o : NB, rest = r - o - nb;
    const int p0 = j / pw * pw * NB;                       // first column of the panel
    const int pe = p0 + pw * NB < r ? p0 + pw * NB : r;    // one past its last column
    rc = chol_step_real(G, L, W, rr, r, o, nb, info, batch, gate, s, pending ? o - NB : -1, pe, pstat);
    pending = false;
    if (rc) return rc;
    if (rest <= 0) break;
    RealGemmDesc<T> u{};
    u.batch = batch;
    u.sA = rr; u.lda = r; u.a_kstrided = 0;
    u.sB = rr; u.ldb = r; u.b_kstrided = 0;
    u.sC = rr; u.ldc = r; u.sE = rr; u.lde = r;
    u.alpha = -1.0; u.beta = 1.0; u.lower_only = 1;
    u.gate = gate.flags; u.gate_want = gate.want;
    if (o + nb < pe) {
      // A small update rides along in the next step's launch, which applies it where it needs it and has
      // workgroups to spare for the rest (one 64 x 64 tile each); a large one is better off as a product of its own.
      long long tiles = 0;
      for (int tc = j + 1; tc * NB < pe; ++tc) tiles += nblk - tc;
      if (defer && (fallback || tiles * batch <= DA_CHOL_DEFER_TILES)) { pending = true; continue; }
      // rest of the panel's columns, all rows from the diagonal down:  A[:, panel] -= L[:, j] L[panel, j]^T
      u.A = L + (long long)(o + nb) * r + o;
      u.B = u.A;
      u.C = G + (long long)(o + nb) * r + (o + nb);
      u.E = u.C;
      u.M = rest; u.N = pe - (o + nb); u.K = nb;
      rc = gemm_real(u, s);
      if (rc) return rc;
    } else {
      // panel done:  A22 -= L[:, panel] L[:, panel]^T, lower triangle only (nothing reads the upper one)
      u.A = L + (long long)pe * r + p0;
      u.B = u.A;
      u.C = G + (long long)pe * r + pe;
      u.E = u.C;
      u.M = r - pe; u.N = r - pe; u.K = pe - p0;
      rc = gemm_real(u, s);
      if (rc) return rc;
    }
  }
  return DA_OK;
}

// P0 <- P0 R^-1 with R = L^T (L, W from chol_factor), in place, `rows` rows per matrix.
template <typename T>
int apply_rinv(T* P0, const T* L, const T* W, int batch, int rows, int r, DaGate gate, hipStream_t s) {
  const int NB = DA_CHOL_NB;
  const int nblk = (r + NB - 1) / NB;
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  const int pw = chol_panel_steps(nblk, gate.flags != nullptr);
  int rc = DA_OK;
  // By the panels of the factorisation: first the solved columns left of the panel are
  // taken out of it in one product,
  //   P0[:, panel] -= P0[:, 0 .. p0] L[panel, 0 .. p0]^T
  // then block column by block column inside it
  //   P0[:, j] <- P0[:, p0 .. j] W[j, p0 .. j]^T
  // (each workgroup owns 64 rows and the one 64-column output tile, and has read all it needs of
  // those rows before it stores)
  for (int j = 0; j < nblk; ++j) {
    const int o = j * NB, nb = r - o < NB ? r - o : NB;
    const int p0 = j / pw * pw * NB;
    const int pe = p0 + pw * NB < r ? p0 + pw * NB : r;
    if (o == p0 && p0 > 0) {
      RealGemmDesc<T> u{};
      u.batch = batch;
      u.A = P0; u.sA = pr; u.lda = r; u.a_kstrided = 0;
      u.B = L + (long long)p0 * r; u.sB = rr; u.ldb = r; u.b_kstrided = 0;
      u.C = P0 + p0; u.sC = pr; u.ldc = r;
      u.E = u.C; u.sE = pr; u.lde = r;
      u.M = rows; u.N = pe - p0; u.K = p0; u.alpha = -1.0; u.beta = 1.0;
      u.gate = gate.flags; u.gate_want = gate.want;
      rc = gemm_real(u, s);
      if (rc) return rc;
    }
    RealGemmDesc<T> a{};
    a.batch = batch;
    a.A = P0 + p0; a.sA = pr; a.lda = r; a.a_kstrided = 0;
    a.B = W + (long long)o * r + p0; a.sB = rr; a.ldb = r; a.b_kstrided = 0;
    a.C = P0 + o; a.sC = pr; a.ldc = r;
    a.E = nullptr;
    a.M = rows; a.N = nb; a.K = o + nb - p0; a.alpha = 1.0; a.beta = 0.0;
    a.gate = gate.flags; a.gate_want = gate.want;
    rc = gemm_real(a, s);
    if (rc) return rc;
  }
  return DA_OK;
}

// One blocked CholeskyQR pass in precision T, in place:  P <- P R^-1  with  P^T P = R^T R.
template <typename T>
int cholqr_pass(T* P0, T* G, T* L, T* W, T* part, int batch, int rows, int r, int r_live, int* info, DaGate gate,
                hipStream_t s, T* pstat = nullptr) {
  int rc = gram<T>(P0, G, part, batch, rows, r, r_live, nullptr, gate, s);
  if (rc) return rc;
  rc = chol_factor<T>(G, L, W, batch, r, info, gate, s, pstat);
  if (rc) return rc;
  return apply_rinv<T>(P0, L, W, batch, rows, r, gate, s);
}

// V = I - up(G - I) for each r x r Gram matrix G of an almost orthonormal P, where up() keeps the strict
// upper triangle and half of the diagonal: the Cholesky factor of G = I + E is R = I + up(E) + O(E^2), so
// P V = P R^-1 + O(E^2).
__global__ __launch_bounds__(256) void polish_factor_kernel(const float* __restrict__ G, float* __restrict__ V,
                                                            long long rr, int r, const int* __restrict__ bad,
                                                            const int* gate, int want) {
  const long long b = blockIdx.y;
  if (!orth_gate_open(gate, want, (int)b)) return;
  const int i = blockIdx.x;
  const float* g = G + b * rr + (long long)i * r;
  float* v = V + b * rr + (long long)i * r;
  const int* bd = bad ? bad + b * r : nullptr;
  const bool row_bad = bd && bd[i];
  for (int j = threadIdx.x; j < r; j += 256) {
    const float x = g[j];
    const bool drop = row_bad || (bd && bd[j]);   // dropped columns neither receive nor give a correction
    v[j] = drop ? (i == j ? 1.f : 0.f) : (i < j ? -x : (i == j ? 1.5f - 0.5f * x : 0.f));
  }
}

// U = up(G - I) in bf16 (see polish_factor_kernel): the factor of the correction product P U, which only has
// to be known to the relative accuracy of bf16 because it is itself of the size of the defect.  Rows and columns
// of dropped columns (`bad`, may be null) are left out of the correction.
// `decide` (if given): every workgroup first evaluates the matrix's verdict after the fp32 pass -- the pass failed or
// left a defect ||P^T P - I||_F above tol (sum of the rows' squared defects, in a fixed order) -- and returns if
// the matrix goes on to the fp64 pass; the workgroup of row 0 records the verdict for the launches that follow.
struct FastVerdict {
  const float* rowdef;
  const int* info32;
  int* need;
  float tol2;
};

__global__ __launch_bounds__(256) void polish_correction_kernel(const float* __restrict__ G, bf16_t* __restrict__ U,
                                                                long long rr, int r, const int* __restrict__ bad,
                                                                const int* gate, int want, FastVerdict decide) {
  const long long b = blockIdx.y;
  if (decide.need) {
    __shared__ float red[256];
    float s = 0.f;
    for (int j = threadIdx.x; j < r; j += 256) s += decide.rowdef[b * r + j];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
      if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
      __syncthreads();
    }
    const bool need = decide.info32[b] != 0 || !(red[0] <= decide.tol2);
    if (blockIdx.x == 0 && threadIdx.x == 0) decide.need[b] = need ? 1 : 0;
    if (need) return;
  } else if (!orth_gate_open(gate, want, (int)b)) {
    return;
  }
  const int i = blockIdx.x;
  const float* g = G + b * rr + (long long)i * r;
  bf16_t* u = U + b * rr + (long long)i * r;
  const int* bd = bad ? bad + b * r : nullptr;
  const bool row_bad = bd && bd[i];
  for (int j = threadIdx.x; j < r; j += 256) {
    const float x = g[j];
    const bool drop = row_bad || (bd && bd[j]);
    u[j] = f2bf(drop ? 0.f : (i < j ? x : (i == j ? 0.5f * (x - 1.f) : 0.f)));
  }
}

// The last polishing pass of an iterate that exists in fp32 and in bf16:  out <- in - in_bf16 U(in^T in), with
// U built from the Gram matrix G (already computed).  The correction product runs on the bf16 matrix cores (its
// relative error 2^-8 times the defect E of `in` adds 4e-3 E to the result, next to the pass's own O(E^2)).
int correction_bf16(const float* in, const bf16_t* in_low, void* out, int out_dtype, const float* G, bf16_t* U,
                    const int* bad, int batch, int rows, int r, DaGate gate, FastVerdict decide, hipStream_t s) {
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  hipLaunchKernelGGL(polish_correction_kernel, dim3((unsigned)r, (unsigned)batch), dim3(256), 0, s, G, U, rr, r, bad,
                     gate.flags, gate.want, decide);
  int rc = da_launch_status();
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
  c.gate = gate.flags; c.gate_want = gate.want;
  return da_gemm_bf16(c, s);
}

// The same in fp32 throughout:  out <- in V(G)  with the triangular V (ranks that are not multiples of 8, and
// intermediate passes).  `in` and `out` are different buffers.
int correction_f32(const float* in, void* out, int out_store, const float* G, float* V, const int* bad, int batch,
                   int rows, int r, DaGate gate, hipStream_t s) {
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  hipLaunchKernelGGL(polish_factor_kernel, dim3((unsigned)r, (unsigned)batch), dim3(256), 0, s, G, V, rr, r, bad,
                     gate.flags, gate.want);
  const int rc = da_launch_status();
  if (rc) return rc;
  // out = in V: V is upper triangular, so column tile j only sums k < 64 (j + 1)
  Gemm32Desc a{};
  a.batch = batch;
  a.A = in; a.sA = pr; a.lda = r; a.a_kstrided = 0;
  a.B = V; a.sB = rr; a.ldb = r; a.b_kstrided = 1;
  a.C = static_cast<float*>(out); a.c_store = out_store; a.sC = pr; a.ldc = r;
  a.M = rows; a.N = r; a.K = r; a.alpha = 1.0; a.beta = 0.0; a.k_tri = 1;
  a.gate = gate.flags; a.gate_want = gate.want;
  return da_gemm_f32s(a, s);
}

int zero_cols(void* out, int dtype, const int* bad, const int* info, int batch, int rows, int r, DaGate gate,
              hipStream_t s) {
  const long long n = (long long)rows * r;
  // (a rare pass: a few workgroups per matrix, so that the launch costs little when no column was dropped)
  long long blocks = (n + 255) / 256;
  const long long cap = 2048 / batch > 8 ? 2048 / batch : 8;
  if (blocks > cap) blocks = cap;
  const dim3 grid((unsigned)blocks, (unsigned)batch);
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(zero_cols_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<bf16_t*>(out), bad, rows, r, info,
                       gate.flags, gate.want);
  else
    hipLaunchKernelGGL(zero_cols_kernel<float>, grid, dim3(256), 0, s, static_cast<float*>(out), bad, rows, r, info,
                       gate.flags, gate.want);
  return da_launch_status();
}

// ---- the fp32 pass on the bf16 matrix cores (bf16 P: its products with bf16 factors are exact in fp32) ----

// G[b] = sum of `n_hh` slabs + sum of `n_hl` slabs and their transposes (the cross terms h^T l + l^T h of a matrix
// held as h + l), in slab order; padded diagonal and row defects as in gram_finish_kernel.  One workgroup per 16 rows:
// it walks the 64-column blocks of its rows, thread t owning row t / 16 and 4 consecutive columns; the transposed
// term comes from the mirrored 64 x 16 tile, read along its rows like the others and turned in LDS.
__global__ __launch_bounds__(256) void gram16_finish_kernel(const float* __restrict__ part, int n_hh, int n_hl,
                                                            long long slab, float* __restrict__ G, long long rr, int r,
                                                            int r_live, float* __restrict__ rowdef, const int* gate,
                                                            int want, int jb_per_z) {
  __shared__ float tr[64][17];
  const int b = blockIdx.y, ib = blockIdx.x;
  if (!orth_gate_open(gate, want, b)) return;
  // gridDim.z > 1: this workgroup covers jb_per_z column blocks and leaves its rows' defects as partial sums,
  // gridDim.y * r floats per z, for rowdef_sum_kernel
  const int jb_first = blockIdx.z * jb_per_z;
  const int ri = threadIdx.x >> 4, c0 = (threadIdx.x & 15) * 4;
  const int mr = threadIdx.x >> 2, mc0 = (threadIdx.x & 3) * 4;
  const int i = ib * 16 + ri;
  const float* pb = part + b * rr;
  const bool vec = (r & 3) == 0;
  float acc = 0.f;
  for (int jb = jb_first; jb < jb_first + jb_per_z && jb * 64 < r; ++jb) {
    const int j0 = jb * 64 + c0;
    float v[4] = {0.f, 0.f, 0.f, 0.f}, m[4] = {0.f, 0.f, 0.f, 0.f};
    if (i < r) {
#pragma unroll 4
      for (int q = 0; q < n_hh + n_hl; ++q) {
        const float* src = pb + q * slab + (long long)i * r + j0;
        if (vec && j0 + 3 < r) {
          const float4 x = *reinterpret_cast<const float4*>(src);
          v[0] += x.x, v[1] += x.y, v[2] += x.z, v[3] += x.w;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (j0 + e < r) v[e] += src[e];
        }
      }
    }
    if (n_hl > 0) {
      // mirrored tile (rows of column block jb, columns of this row block), summed over the cross-term slabs
      const int mj = jb * 64 + mr, mi0 = ib * 16 + mc0;
      if (mj < r) {
#pragma unroll 4
        for (int q = n_hh; q < n_hh + n_hl; ++q) {
          const float* src = pb + q * slab + (long long)mj * r + mi0;
          if (vec && mi0 + 3 < r) {
            const float4 x = *reinterpret_cast<const float4*>(src);
            m[0] += x.x, m[1] += x.y, m[2] += x.z, m[3] += x.w;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (mi0 + e < r) m[e] += src[e];
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 4; ++e) tr[mr][mc0 + e] = m[e];
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += tr[c0 + e][ri];
    }
    if (i < r) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int j = j0 + e;
        if (j < r) {
          if (i >= r_live && j == i) v[e] = 1.f;
          const float d = v[e] - (i == j ? 1.f : 0.f);
          acc += d * d;
        }
      }
      float* dst = G + b * rr + (long long)i * r + j0;
      if (vec && j0 + 3 < r) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (j0 + e < r) dst[e] = v[e];
      }
    }
  }
  if (rowdef) {
    // the sixteen threads of a row sit in one wavefront
    for (int o = 1; o < 16; o <<= 1) acc += __shfl_xor(acc, o);
    if ((threadIdx.x & 15) == 0 && i < r) rowdef[((long long)blockIdx.z * gridDim.y + b) * r + i] = acc;
  }
}

// rowdef[e] = part[0][e] + part[1][e] + ... in that order (`n` floats per part)
__global__ __launch_bounds__(256) void rowdef_sum_kernel(const float* __restrict__ part, int parts, long long n,
                                                         float* __restrict__ rowdef) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  float s = 0.f;
  for (int z = 0; z < parts; ++z) s += part[z * n + e];
  rowdef[e] = s;
}

// G = H^T H (+ H^T Lo + Lo^T H when Lo is given), fp32, from bf16 operands: the two products run as the groups of
// one launch, each cut into K slices that are tiles of their own (so that a tall, narrow H still fills the GPU),
// and leave fp32 slabs that the finish kernel adds in order.
int gram16(const bf16_t* H, const bf16_t* Lo, float* G, float* part, int batch, int rows, int r, int r_live,
           float* rowdef, float* rowdef_part, DaGate gate, hipStream_t s) {
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  const int kinds = Lo ? 2 : 1;
  int ks = 0;
  const int nsl = gram16_slices(batch, rows, r, kinds, &ks);
  GemmDesc g[2];
  const int n = kinds;
  for (int kind = 0; kind < kinds; ++kind) {
    GemmDesc& d = g[kind];
    d = GemmDesc{};
    d.batch = batch;
    d.A = H; d.sA = pr; d.lda = r; d.a_kstrided = 1;
    d.B = kind == 0 ? H : Lo; d.sB = pr; d.ldb = r; d.b_kstrided = 1;
    // the slices' partial products: slabs kind * nsl ... kind * nsl + nsl - 1 of `batch` matrices each
    d.C = part + (long long)kind * nsl * rr * batch; d.sC = rr; d.ldc = r; d.c_dtype = DA_F32;
    d.M = r; d.N = r; d.K = rows;
    d.k_slices = nsl; d.k_slice = ks;
    d.epilogue = DA_EPI_STORE; d.s1 = 1.f; d.faithful = 0;
    d.gate = gate.flags; d.gate_want = gate.want;
  }
  int rc = da_gemm_bf16_grouped(g, n, s);
  if (rc) return rc;
  // few row blocks (a narrow factor, a small batch): one workgroup per column block as well, so that the slabs are
  // read by enough workgroups; the rows' defects then take a second, tiny launch
  const int njb = (r + 63) / 64, row_wgs = (r + 15) / 16 * batch;
  const int nz = row_wgs < 256 ? njb : 1;
  hipLaunchKernelGGL(gram16_finish_kernel, dim3((unsigned)((r + 15) / 16), (unsigned)batch, (unsigned)nz), dim3(256), 0, s,
                     part, nsl, Lo ? nsl : 0, rr * batch, G, rr, r, r_live, rowdef && nz > 1 ? rowdef_part : rowdef,
                     gate.flags, gate.want, nz > 1 ? 1 : njb);
  rc = da_launch_status();
  if (rc || !rowdef || nz == 1) return rc;
  const long long nd = (long long)batch * r;
  hipLaunchKernelGGL(rowdef_sum_kernel, dim3((unsigned)((nd + 255) / 256)), dim3(256), 0, s, rowdef_part, nz, nd, rowdef);
  return da_launch_status();
}

// T = identity (r x r per matrix)
__global__ __launch_bounds__(256) void eye_kernel(float* __restrict__ T, long long rr, int r) {
  const long long b = blockIdx.y;
  const int i = blockIdx.x;
  for (int j = threadIdx.x; j < r; j += 256) T[b * rr + (long long)i * r + j] = i == j ? 1.f : 0.f;
}

// Tcat[k][0 .. r) = bf16(T[k][:]), Tcat[k][r .. 2r) = bf16(T[k][:] - that): T to 16 bits as two bf16 factors
// `stacked`: [T_hi; T_lo] (2r x r) instead of [T_hi | T_lo] (r x 2r).  `lower`: the source holds L^-1 (lower
// triangular, blocks of 64 above the diagonal never written) and T = R^-1 is its transpose.
__global__ __launch_bounds__(256) void split_factor_kernel(const float* __restrict__ T, bf16_t* __restrict__ Tcat,
                                                           long long rr, int r, int stacked, int lower) {
  const long long b = blockIdx.y;
  const int k = blockIdx.x;
  const float* t = T + b * rr + (long long)k * r;
  bf16_t* o = Tcat + b * 2 * rr + (long long)k * (stacked ? r : 2 * r);
  const long long lo = stacked ? rr : r;
  for (int j = threadIdx.x; j < r; j += 256) {
    const float v = !lower ? t[j] : ((j >> 6) >= (k >> 6) ? T[b * rr + (long long)j * r + k] : 0.f);
    const bf16_t h = f2bf(v);
    o[j] = h;
    o[lo + j] = f2bf(v - bf2f(h));
  }
}

// C2 (rows x 2r, fp32) holds P T_hi | P T_lo: their sum as h + l (two bf16 matrices, 16 bits together)
__global__ __launch_bounds__(256) void split_sum_kernel(const float* __restrict__ C2, bf16_t* __restrict__ H,
                                                        bf16_t* __restrict__ Lo, long long pr, int r) {
  const long long b = blockIdx.y;
  const float* c = C2 + b * 2 * pr;
  for (long long e = ((long long)blockIdx.x * 256 + threadIdx.x) * 4; e < pr; e += (long long)gridDim.x * 1024) {
    const long long row = e / r;
    const int col = (int)(e - row * r);   // r is a multiple of 8: the four elements share the row
    const float4 a = *reinterpret_cast<const float4*>(c + row * 2 * r + col);
    const float4 d = *reinterpret_cast<const float4*>(c + row * 2 * r + r + col);
    const float v[4] = {a.x + d.x, a.y + d.y, a.z + d.z, a.w + d.w};
    bf16_t h[4], l[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      h[q] = f2bf(v[q]);
      l[q] = f2bf(v[q] - bf2f(h[q]));
    }
    *reinterpret_cast<uint2*>(H + b * pr + e) = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
    *reinterpret_cast<uint2*>(Lo + b * pr + e) = make_uint2((uint32_t)l[0] | ((uint32_t)l[1] << 16), (uint32_t)l[2] | ((uint32_t)l[3] << 16));
  }
}

// The fp32 CholeskyQR pass of a bf16 P with its large products on the bf16 matrix cores:
//   G = P^T P (exact products, fp32 sums), blocked Cholesky G = R^T R in fp32, T = R^-1 explicitly (the block
//   recurrence of the triangular solve applied to the identity), P1 = P T with T as two bf16 factors (T to 16
//   bits: P1 stays an exact triangular recombination of P's columns, so its thin-QR factor is P's), kept as
//   h + l (bf16 each); then G2 = P1^T P1 = h^T h + h^T l + l^T h for the defect and the polishing pass.
int fast16_pass(const bf16_t* P, const OrthWs& w, int batch, int rows, int r, int r_live, bool second_gram,
                hipStream_t s) {
  const int NB = DA_CHOL_NB;
  const int nblk = (r + NB - 1) / NB;
  const long long pr = (long long)rows * r, rr = (long long)r * r;
  const DaGate all{nullptr, 0};
  float* G = reinterpret_cast<float*>(w.G);
  float* L = reinterpret_cast<float*>(w.L);
  float* W = reinterpret_cast<float*>(w.W);
  float* T = W + rr * batch;                          // second half of W's room
  bf16_t* Tcat = reinterpret_cast<bf16_t*>(w.L);      // over the factor L, which is dead once W is complete
  float* C2 = reinterpret_cast<float*>(w.P0);         // rows x 2r fp32 = the room of the fp64 copy
  bf16_t* Lo = reinterpret_cast<bf16_t*>(w.Pf);
  float* part = reinterpret_cast<float*>(w.part);
  int rc = gram16(P, nullptr, G, part, batch, rows, r, r_live, nullptr, nullptr, all, s);
  if (rc) return rc;
  // (the steps write the rows of L^-1 themselves: no W, no recurrence on the identity afterwards)
  static const bool inv_rows = [] { const char* e = getenv("DION_AMD_ORTH_NO_INV"); return !(e && atoi(e)); }();
  // (every step's trailing update rides along in the next step's launch)
  static const bool defer = [] { const char* e = getenv("DION_AMD_CHOL_NO_DEFER"); return !(e && atoi(e)); }();
  static const bool lag_on = [] { const char* e = getenv("DION_AMD_CHOL_NO_TLAG"); return !(e && atoi(e)); }();
  const bool lag = inv_rows && lag_on && nblk >= 4;   // (short chains: the extra launch at the end costs what the lag saves)
  bool pending = false;
  for (int j = 0; j < nblk; ++j) {
    const int o = j * NB, nb = r - o < NB ? r - o : NB, rest = r - o - nb;
    const int o_prev = pending ? o - NB : -1;
    // (the rows of L^-1 lag one step behind: row j - 1 is formed by workgroups of step j's launch that do nothing else)
    rc = inv_rows ? da_chol_step_f32_inv(G, L, T, rr, r, o, nb, w.info32, batch, all, s, o_prev, r,
                                         lag && j >= 2 ? j - 1 : -1, lag ? 0 : 1)
                  : da_chol_step_f32(G, L, W, rr, r, o, nb, w.info32, batch, all, s, o_prev, r);
    pending = false;
    if (rc) return rc;
    if (rest <= 0) break;
    // (small updates only: see cholqr_pass)
    const long long below = nblk - j - 1;
    if (defer && below * (below + 1) / 2 * batch <= DA_CHOL_DEFER_TILES) { pending = true; continue; }
    Gemm32Desc u{};
    u.batch = batch;
    u.A = L + (long long)(o + nb) * r + o; u.sA = rr; u.lda = r; u.a_kstrided = 0;
    u.B = u.A; u.sB = rr; u.ldb = r; u.b_kstrided = 0;
    u.C = G + (long long)(o + nb) * r + (o + nb); u.sC = rr; u.ldc = r;
    u.E = u.C; u.sE = rr; u.lde = r;
    u.M = rest; u.N = rest; u.K = nb; u.alpha = -1.0; u.beta = 1.0; u.lower_only = 1;
    rc = da_gemm_f32s(u, s);
    if (rc) return rc;
  }
  if (lag) {
    rc = da_chol_trow_f32(L, T, rr, r, nblk - 1, batch, all, s);
    if (rc) return rc;
  }
  if (!inv_rows) {
    hipLaunchKernelGGL(eye_kernel, dim3((unsigned)r, (unsigned)batch), dim3(256), 0, s, T, rr, r);
    rc = da_launch_status();
    if (rc) return rc;
  }
  for (int j = 0; j < nblk && !inv_rows; ++j) {
    const int o = j * NB, nb = r - o < NB ? r - o : NB;
    Gemm32Desc a{};
    a.batch = batch;
    a.A = T; a.sA = rr; a.lda = r; a.a_kstrided = 0;
    a.B = W + (long long)o * r; a.sB = rr; a.ldb = r; a.b_kstrided = 0;
    a.C = T + o; a.sC = rr; a.ldc = r;
    // rows below block j of T are zero in these columns (T is upper triangular): only rows < o + nb are needed
    a.M = o + nb; a.N = nb; a.K = o + nb; a.alpha = 1.0; a.beta = 0.0;
    rc = da_gemm_f32s(a, s);
    if (rc) return rc;
  }
  // P1 = P T_hi + P T_lo.  With whole 64-deep stages (r a multiple of 64) it is ONE accumulation over the stacked
  // factor [T_hi; T_lo], P read twice along k, and the product leaves the kernel as h + l; otherwise the two
  // products go side by side into an fp32 matrix and a pass of its own adds and splits them.
  const bool stacked = r % 64 == 0 && rows % 128 == 0 && (Lo - w.Ph) % 8 == 0;
  hipLaunchKernelGGL(split_factor_kernel, dim3((unsigned)r, (unsigned)batch), dim3(256), 0, s, T, Tcat, rr, r,
                     stacked ? 1 : 0, inv_rows ? 1 : 0);
  rc = da_launch_status();
  if (rc) return rc;
  if (stacked) {
    GemmDesc c{};
    c.batch = batch;
    c.A = P; c.sA = pr; c.lda = r; c.a_kstrided = 0; c.a_kwrap = r;
    c.B = Tcat; c.sB = 2 * rr; c.ldb = r; c.b_kstrided = 1;
    c.C = w.Ph; c.sC = pr; c.ldc = r; c.c_dtype = DA_BF16; c.c2_off = Lo - w.Ph;
    c.M = rows; c.N = r; c.K = 2 * r;
    c.epilogue = DA_EPI_STORE; c.s1 = 1.f; c.faithful = 0;
    rc = da_gemm_bf16(c, s);
    if (rc || !second_gram) return rc;
    return gram16(w.Ph, Lo, G, part, batch, rows, r, r_live, w.rowdef, w.rowdef_part, all, s);
  }
  GemmDesc c{};
  c.batch = batch;
  c.A = P; c.sA = pr; c.lda = r; c.a_kstrided = 0;
  c.B = Tcat; c.sB = 2 * rr; c.ldb = 2 * r; c.b_kstrided = 1;
  c.C = C2; c.sC = 2 * pr; c.ldc = 2 * r; c.c_dtype = DA_F32;
  c.M = rows; c.N = 2 * r; c.K = r;
  c.epilogue = DA_EPI_STORE; c.s1 = 1.f; c.faithful = 0;
  rc = da_gemm_bf16(c, s);
  if (rc) return rc;
  long long blocks = (pr / 4 + 255) / 256;
  const long long cap = 16384 / batch > 0 ? 16384 / batch : 1;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(split_sum_kernel, dim3((unsigned)(blocks < 1 ? 1 : blocks), (unsigned)batch), dim3(256), 0, s, C2,
                     w.Ph, Lo, pr, r);
  rc = da_launch_status();
  if (rc || !second_gram) return rc;
  return gram16(w.Ph, Lo, G, part, batch, rows, r, r_live, w.rowdef, w.rowdef_part, all, s);
}

// After the fp64 factorisation: which of the matrices it ran for need the polishing pass.  The pivots are the
// squares of R's diagonal, so pmax / pmin <= cond(R)^2 = cond(P)^2; with pmin >= ratio * pmax and no failed pivot the
// defect the fp64 pass leaves, eps64 * cond(P)^2, is far below what the result's dtype resolves even if cond(P) is
// a hundred times the estimate, and the result is converted as it is.
__global__ void decide_polish_kernel(const double* __restrict__ pstat, const int* __restrict__ info,
                                     const int* gate, int want, int* __restrict__ polish, int* __restrict__ direct,
                                     int batch, double ratio) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch) return;
  const bool open = orth_gate_open(gate, want, b);
  const double mn = pstat[2 * b], mx = pstat[2 * b + 1];
  const bool healthy = info[b] == 0 && mn >= ratio * mx && mx > 0.0;   // (false for NaN)
  polish[b] = open && !healthy ? 1 : 0;
  direct[b] = open && healthy ? 1 : 0;
}

// bf16 copy of the matrices whose gate is open
__global__ __launch_bounds__(256) void copy_bf16_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst,
                                                        long long per, const int* gate, int want) {
  const long long b = blockIdx.y;
  if (!orth_gate_open(gate, want, (int)b)) return;
  const uint4* s4 = reinterpret_cast<const uint4*>(src + b * per);
  uint4* d4 = reinterpret_cast<uint4*>(dst + b * per);
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < per / 8; i += (long long)gridDim.x * 256) d4[i] = s4[i];
}

// need[b] = the fp32 factorisation of matrix b met a pivot that was not positive
__global__ void decide_cqr_kernel(const int* __restrict__ info32, int* __restrict__ need, int batch) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < batch) need[b] = info32[b] != 0 ? 1 : 0;
}

// Defect ||P^T P - I||_F up to which the closed-form polishing pass is trusted after the fp32 pass: it leaves
// about 3 E^2, i.e. 1e-5.
constexpr float FAST_TOL = 2e-3f;
// Smallest pivot, relative to the largest, with which the fp64 pass's result needs no polishing pass: the pivot range
// then puts cond(P) at 3e3 or more below, eps64 * cond^2 at 1e-9 -- and at 1e-5 if the estimate is a hundred times
// too low.
constexpr double POLISH_PIVOT_RATIO = 1e-7;

}  // namespace

// Thin-QR Q factor of each P (same column space, orthonormal columns, up to column signs).
//   passes == 2 (the optimizer's case): a blocked CholeskyQR pass in fp32, the Gram matrix of its result (which
//   measures the defect E = ||P^T P - I||_F it left: eps32 * cond(P)^2) and, for a small defect, the closed form of
//   a second CholeskyQR pass: R^-1 = I - up(P^T P - I) + O(E^2).  Matrices for which the fp32 pass failed or left
//   too large a defect are flagged on the device, and the same sequence in fp64 then runs for those alone (every
//   launch of it returns at once for the others; no host synchronisation): the Gram matrix squares P's condition
//   number, up to 4e12 on the optimizer's full-rank inputs.  After the fp64 pass, columns whose row of
//   P^T P - I is not small came from pivots at round-off level (a numerically rank-deficient P): they are zeroed
//   and reported in `info` like a non-positive pivot.
//   passes == 1: the fp64 pass alone.  passes == 3: fp64 pass and two polishing passes.
// Columns r_live .. r-1 of P, if any, must be zero on entry and are zero on return (a caller pads the
// rank to a multiple of 8 this way); the polishing passes multiply them by finite factors only.
int da_orthonormalize(const void* P, void* out, int dtype, int batch, int rows, int r, int r_live, int passes,
                      int method, void* ws, int* info, hipStream_t s) {
  if (passes < 1 || batch > 65535 || r_live < 1 || r_live > r || r - r_live > 63) return DA_ERR_ARG;
  if (method != DA_QR_AUTO && method != DA_QR_FP64 && method != DA_QR_CQR) return DA_ERR_ARG;
  const long long pr = (long long)rows * r;
  const OrthWs w(ws, batch, rows, r);
  static const bool force64 = getenv("DION_AMD_ORTH_FP64") != nullptr;
  const bool low = (r & 7) == 0;   // the bf16 correction product moves 16-byte chunks
  // (a P that is square or nearly so is a full-rank factor: its condition number is beyond fp32 as a rule)
  const bool cqr = passes == 2 && method == DA_QR_CQR;
  const bool fast = cqr || (passes == 2 && method == DA_QR_AUTO && !force64 && rows >= 4 * r);
  static const bool no16 = getenv("DION_AMD_ORTH_NO_BF16") != nullptr;
  // (the Gram products on the bf16 matrix cores sum over the rows in 16-byte chunks: rows a multiple of 8 as well;
  // other factors keep the fp32 kernels, which take any number of rows)
  const bool rows8 = (rows & 7) == 0;
  const bool fast16 = fast && dtype == DA_BF16 && low && rows8 && !no16;
  const DaGate all{nullptr, 0};
  int rc;
  if (cqr) {
    // ---- "cqr": the fp32 CholeskyQR pass is the result (reference dion/dion_reference.py:752-758)
    if (fast16) {
      rc = fast16_pass(static_cast<const bf16_t*>(P), w, batch, rows, r, r_live, false, s);
    } else {
      rc = da_cvt_to_f32(P, dtype, w.Pf, pr, batch, all, s);
      if (rc) return rc;
      rc = cholqr_pass<float>(w.Pf, reinterpret_cast<float*>(w.G), reinterpret_cast<float*>(w.L),
                              reinterpret_cast<float*>(w.W), reinterpret_cast<float*>(w.part), batch, rows, r, r_live,
                              w.info32, all, s);
    }
    if (rc) return rc;
    hipLaunchKernelGGL(decide_cqr_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, w.info32, w.need, batch);
    rc = da_launch_status();
    if (rc) return rc;
    const DaGate good{w.need, 0};
    if (fast16) {
      long long blocks = (pr / 8 + 255) / 256;
      if (blocks > 1024) blocks = 1024;
      hipLaunchKernelGGL(copy_bf16_kernel, dim3((unsigned)(blocks < 1 ? 1 : blocks), (unsigned)batch), dim3(256), 0, s, w.Ph,
                         static_cast<bf16_t*>(out), pr, good.flags, good.want);
      rc = da_launch_status();
    } else {
      rc = da_cvt_from_f32(w.Pf, out, dtype, pr, batch, good, s);
    }
    if (rc) return rc;
  } else if (fast) {
    // ---- fp32 pass on every matrix
    float* G = reinterpret_cast<float*>(w.G);
    float* L = reinterpret_cast<float*>(w.L);
    float* W = reinterpret_cast<float*>(w.W);
    if (fast16) {
      rc = fast16_pass(static_cast<const bf16_t*>(P), w, batch, rows, r, r_live, true, s);
      if (rc) return rc;
    } else {
      rc = da_cvt_to_f32(P, dtype, w.Pf, pr, batch, all, s);
      if (rc) return rc;
      rc = cholqr_pass<float>(w.Pf, G, L, W, reinterpret_cast<float*>(w.part), batch, rows, r, r_live, w.info32, all, s);
      if (rc) return rc;
      if (low) {
        rc = da_cvt_f32_to_bf16(w.Pf, w.Ph, pr, batch, all, s);
        if (rc) return rc;
      }
      rc = gram<float>(w.Pf, G, reinterpret_cast<float*>(w.part), batch, rows, r, r_live, w.rowdef, all, s);
      if (rc) return rc;
    }
    const DaGate good{w.need, 0};
    if (low) {
      // (the verdict is part of the correction factor's launch)
      const FastVerdict verdict{w.rowdef, w.info32, w.need, FAST_TOL * FAST_TOL};
      rc = correction_bf16(w.Pf, w.Ph, out, dtype, G, reinterpret_cast<bf16_t*>(L), nullptr, batch, rows, r, good, verdict, s);
    } else {
      hipLaunchKernelGGL(decide_fast_kernel, dim3((unsigned)batch), dim3(64), 0, s, w.rowdef, w.info32, w.need, r,
                         FAST_TOL * FAST_TOL);
      rc = da_launch_status();
      if (rc) return rc;
      rc = correction_f32(w.Pf, out, da_store_of(dtype), G, L, nullptr, batch, rows, r, good, s);
    }
    if (rc) return rc;
  }
  // ---- fp64 pass: on the flagged matrices, or on all of them
  const DaGate gate = fast ? DaGate{w.need, 1} : all;
  rc = da_cvt_to_f64(P, dtype, w.P0, pr, batch, gate, s);
  if (rc) return rc;
  rc = cholqr_pass<double>(w.P0, w.G, w.L, w.W, w.part, batch, rows, r, r_live, info, gate, s, w.pstat);
  if (rc) return rc;
  if (passes == 1) return da_cvt_from_f64(w.P0, out, dtype, pr, batch, gate, s);
  // One polishing pass (the optimizer's case) is for factors whose conditioning leaves a visible defect even in fp64
  // and for noise-level pivots: the pivot range tells on the device which matrices those are; the others are done.
  // (not as the fall-back of an fp32 pass: those matrices were flagged for their conditioning, and the launches that
  // find nothing to do should be few)
  static const bool always_polish_env = getenv("DION_AMD_ORTH_ALWAYS_POLISH") != nullptr;
  const bool always_polish = always_polish_env || fast;
  const DaGate whole = gate;   // every matrix of the fp64 pass
  if (passes == 2 && !always_polish) {
    hipLaunchKernelGGL(decide_polish_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, w.pstat, info, gate.flags,
                       gate.want, w.polish, w.direct, batch, POLISH_PIVOT_RATIO);
    rc = da_launch_status();
    if (rc) return rc;
    rc = da_cvt_from_f64(w.P0, out, dtype, pr, batch, DaGate{w.direct, 1}, s);
    if (rc) return rc;
  }
  const DaGate gate2 = passes == 2 && !always_polish ? DaGate{w.polish, 1} : whole;
  float* Gf = reinterpret_cast<float*>(w.G);
  const bool last_low = passes == 2 && low;
  // A bf16 result after one polishing pass needs the fp64 pass's result to 16 bits only, as h + l (bf16 each): the
  // Gram matrix that measures its defect then runs on the bf16 matrix cores (h^T h + h^T l + l^T h), and the
  // correction product reads h.  Otherwise: one conversion pass to fp32 costs less than reading fp64 twice in the
  // polishing products.
  const bool hl = last_low && dtype == DA_BF16 && rows8 && !no16;
  bf16_t* Lo = reinterpret_cast<bf16_t*>(w.Pf);
  rc = hl ? da_cvt_f64_to_hl(w.P0, w.Ph, Lo, pr, batch, gate2, s)
          : da_cvt_f64_to_f32(w.P0, w.Pf, last_low ? w.Ph : nullptr, pr, batch, gate2, s);
  if (rc) return rc;
  const float* cur = w.Pf;
  for (int pass = 1; pass < passes; ++pass) {
    const bool last = pass + 1 == passes;
    rc = hl ? gram16(w.Ph, Lo, Gf, reinterpret_cast<float*>(w.part), batch, rows, r, r_live, w.rowdef, w.rowdef_part, gate2, s)
            : gram<float>(cur, Gf, reinterpret_cast<float*>(w.part), batch, rows, r, r_live, w.rowdef, gate2, s);
    if (rc) return rc;
    const int* bad = nullptr;
    if (pass == 1) {
      hipLaunchKernelGGL(decide_cols_kernel, dim3((unsigned)batch), dim3(256), 0, s, w.rowdef, w.bad, info, r,
                         gate2.flags, gate2.want);
      rc = da_launch_status();
      if (rc) return rc;
      bad = w.bad;
    }
    if (last && last_low) {
      rc = correction_bf16(cur, w.Ph, out, dtype, Gf, reinterpret_cast<bf16_t*>(w.L), bad, batch, rows, r, gate2,
                           FastVerdict{nullptr, nullptr, nullptr, 0.f}, s);
    } else {
      // intermediate iterates alternate between the fp32 buffer and (as fp32) the no longer needed P0
      float* other = cur == w.Pf ? reinterpret_cast<float*>(w.P0) : w.Pf;
      rc = correction_f32(cur, last ? out : static_cast<void*>(other), last ? da_store_of(dtype) : DA_STORE_NATIVE, Gf,
                          reinterpret_cast<float*>(w.L), bad, batch, rows, r, gate2, s);
      cur = other;
    }
    if (rc) return rc;
  }
  return zero_cols(out, dtype, w.bad, info, batch, rows, r, gate2, s);
}

// Scratch of da_orthonormalize_sketch beyond da_orth_workspace_bytes: S P in the factor's dtype and in fp64.
size_t da_orth_sketch_extra_bytes(int batch, int k, int r) {
  const size_t kr = (size_t)batch * k * r;
  return orth_align(kr * 4) + orth_align(kr * 8) + 256;
}

// The reference's randomised Cholesky QR with the sketch S given by the caller (reference dion/dion.py:1287-1303):
//   SP = S P (in P's dtype);  R1 = R-factor of SP;  P1 = P R1^-1;  R2 = chol(P1^T P1);  Q = P1 R2^-1.
// R1 is taken as the Cholesky factor of (SP)^T (SP) formed in fp64 -- the R-factor of a Householder QR of SP up to
// the signs of its rows, which P1's column space does not see -- and both triangular solves and the second
// factorisation run in fp64 as well (the reference's are fp32).  rows <= r: the reference factors such a P by
// Householder QR without a sketch (1283-1285); here: the fp64 pass.
int da_orthonormalize_sketch(const void* P, const void* S, void* out, int dtype, int batch, int rows, int r, int r_live,
                             int k, void* ws, void* extra, int* info, hipStream_t s) {
  if (rows <= r_live) return da_orthonormalize(P, out, dtype, batch, rows, r, r_live, 2, DA_QR_FP64, ws, info, s);
  if (!S || !extra || k < r_live || batch > 65535 || r_live < 1 || r_live > r || r - r_live > 63) return DA_ERR_ARG;
  const long long pr = (long long)rows * r, kr = (long long)k * r, ks = (long long)k * rows;
  const OrthWs w(ws, batch, rows, r);
  const DaGate all{nullptr, 0};
  char* x = static_cast<char*>(extra);
  void* SPlow = x;
  double* SP = reinterpret_cast<double*>(x + orth_align((size_t)batch * kr * 4));
  // ---- SP = S P, rounded to the factor's dtype as the reference's matmul does
  GemmDesc g{};
  g.batch = batch;
  g.A = S; g.sA = ks; g.lda = rows; g.a_kstrided = 0;
  g.B = P; g.sB = pr; g.ldb = r; g.b_kstrided = 1;
  g.C = SPlow; g.sC = kr; g.ldc = r; g.c_dtype = dtype;
  g.M = k; g.N = r; g.K = rows;
  g.epilogue = DA_EPI_STORE; g.s1 = 1.f; g.faithful = 0;
  int rc = dtype == DA_BF16 ? da_gemm_bf16(g, s) : da_gemm_f32(g, s);
  if (rc) return rc;
  rc = da_cvt_to_f64(SPlow, dtype, SP, kr, batch, all, s);
  if (rc) return rc;
  // ---- R1^T R1 = (SP)^T (SP)
  rc = gram<double>(SP, w.G, w.part, batch, k, r, r_live, nullptr, all, s, true);
  if (rc) return rc;
  rc = chol_factor<double>(w.G, w.L, w.W, batch, r, info, all, s);
  if (rc) return rc;
  // ---- P1 = P R1^-1
  rc = da_cvt_to_f64(P, dtype, w.P0, pr, batch, all, s);
  if (rc) return rc;
  rc = apply_rinv<double>(w.P0, w.L, w.W, batch, rows, r, all, s);
  if (rc) return rc;
  // ---- Cholesky QR of the preconditioned factor
  rc = cholqr_pass<double>(w.P0, w.G, w.L, w.W, w.part, batch, rows, r, r_live, info, all, s);
  if (rc) return rc;
  return da_cvt_from_f64(w.P0, out, dtype, pr, batch, all, s);
}

