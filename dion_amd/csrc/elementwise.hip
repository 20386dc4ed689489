// HBM-bound passes around the Newton-Schulz iteration (all single-pass, 16-byte accesses):
//
//   stage_wide  : source matrix -> bf16/f32 working matrix in *wide* orientation
//                 (rows <= cols; tall sources are transposed through an LDS tile), fused
//                 with either a plain dtype cast (stand-alone Newton-Schulz) or Muon's
//                 momentum / Nesterov update, plus per-tile partial sums of squares for
//                 the Frobenius norm.
//   norm_finish : fixed-order reduction of the partial sums -> divisor per matrix.
//   normalize   : X <- X / (||X||_F + eps) with the reference's rounding points.
//   unstage     : wide working matrix -> destination orientation; either a plain store
//                 (stand-alone Newton-Schulz) or Muon's weight-decay + scaled update.
//
// Rounding follows the reference op by op (reference dion/muon.py:536-550, 569-573,
// 633-638); the translation unit must be compiled with -ffp-contract=off.
#include "common.h"
#include "elementwise.h"

namespace {

constexpr int TS = 64;  // tile edge of the transposing passes; 256 threads, 16 elements (two 8-wide chunks) per thread
constexpr int RT = 32, CT = 256;   // tile of the passes that keep the orientation: 32 rows x 256 columns

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = bf2f((bf16_t)(w[i] & 0xffffu));
      v[2 * i + 1] = bf2f((bf16_t)(w[i] >> 16));
    }
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f2bf(v[2 * i]) | ((uint32_t)f2bf(v[2 * i + 1]) << 16);
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  // streaming variants: data that is not touched again before it would fall out of the caches anyway
  static __device__ __forceinline__ void load_nt(const bf16_t* p, float (&v)[8]) {
    typedef unsigned u4_t __attribute__((ext_vector_type(4)));
    const u4_t w = __builtin_nontemporal_load(reinterpret_cast<const u4_t*>(p));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned x = w[i];
      v[2 * i] = __builtin_bit_cast(float, x << 16);
      v[2 * i + 1] = __builtin_bit_cast(float, x & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store_nt(bf16_t* p, const float (&v)[8]) {
    typedef unsigned u4_t __attribute__((ext_vector_type(4)));
    u4_t w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f2bf(v[2 * i]) | ((uint32_t)f2bf(v[2 * i + 1]) << 16);
    __builtin_nontemporal_store(w, reinterpret_cast<u4_t*>(p));
  }
  static __device__ __forceinline__ float round(float x) { return rbf(x); }
};
template <> struct Vec8<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
  static __device__ __forceinline__ void load_nt(const float* p, float (&v)[8]) {
    typedef float f4_t __attribute__((ext_vector_type(4)));
    const f4_t a = __builtin_nontemporal_load(reinterpret_cast<const f4_t*>(p));
    const f4_t b = __builtin_nontemporal_load(reinterpret_cast<const f4_t*>(p) + 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float x = a[i], y = b[i];
      v[i] = x;
      v[4 + i] = y;
    }
  }
  static __device__ __forceinline__ void store_nt(float* p, const float (&v)[8]) {
    typedef float f4_t __attribute__((ext_vector_type(4)));
    const f4_t a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
    __builtin_nontemporal_store(a, reinterpret_cast<f4_t*>(p));
    __builtin_nontemporal_store(b, reinterpret_cast<f4_t*>(p) + 1);
  }
  static __device__ __forceinline__ float round(float x) { return x; }
};

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
  if (threadIdx.x == 0) s = (red[0] + red[1]) + (red[2] + red[3]);
  return s;  // valid in thread 0
}

// ---------------------------------------------------------------------------------------
// stage_wide
// ---------------------------------------------------------------------------------------
// Source element access, in the source's own (rows x cols, row-major) orientation.
template <typename TG, typename TM, typename TW>
struct StageArgs {
  DaPtrTable g;       // sources (gradients), one pointer per matrix
  DaPtrTable mom;     // momentum buffers (Muon mode), modified in place; unused for plain
  TW* wide;           // [batch][mw][ldw], columns < nw used
  float* partials;    // [batch][tiles]
  int rows, cols;     // source shape
  int ld;             // source row pitch (elements)
  int ldw;            // row pitch of the wide matrices (elements)
  float mu;
  int nesterov;
  int muon;           // 1: momentum update, 0: plain cast
  int use_wtab;       // 1: result b goes to wtab.p[b] (rows x cols contiguous); never with TALL
  DaPtrTable wtab;
};

template <typename TG, typename TM, typename TW, bool TALL>
__global__ __launch_bounds__(256) void stage_wide_kernel(StageArgs<TG, TM, TW> a) {
  // Tile coordinates are in the source orientation: tile (ti, tj) covers source rows
  // ti*64.., cols tj*64...  The wide matrix is the source (TALL = false) or its transpose.
  __shared__ float red[4];
  __shared__ float tile[TALL ? TS : 1][TS + 1];
  const int b = blockIdx.y;
  const int tiles_c = (a.cols + TS - 1) / TS;
  const int ti = blockIdx.x / tiles_c, tj = blockIdx.x % tiles_c;
  const int tid = threadIdx.x;
  const TG* G = static_cast<const TG*>(a.g.p[b]);
  TM* M = a.muon ? static_cast<TM*>(a.mom.p[b]) : nullptr;
  const int mw = TALL ? a.cols : a.rows, nw = TALL ? a.rows : a.cols;
  TW* W = a.use_wtab ? static_cast<TW*>(a.wtab.p[b]) : a.wide + (long long)b * mw * a.ldw;

  float ss = 0.f;
  if (!TALL) {
    // No transpose: a tile is RT rows x CT columns, a wavefront's 16-byte accesses cover whole 512-byte row
    // segments, and all of a thread's loads are requested before the first is used.
    const int tiles_cw = (a.cols + CT - 1) / CT;
    const int wi = blockIdx.x / tiles_cw, wj = blockIdx.x % tiles_cw;
    constexpr int NC = RT * CT / 8 / 256;   // chunks per thread
    float g[NC][8], m[NC][8];
    bool ok[NC];
#pragma unroll
    for (int it = 0; it < NC; ++it) {
      const int c = tid + 256 * it;
      const int i = wi * RT + c / (CT / 8), j = wj * CT + (c % (CT / 8)) * 8;
      ok[it] = i < a.rows && j < a.cols;
      if (ok[it]) {
        Vec8<TG>::load_nt(G + (long long)i * a.ld + j, g[it]);
        if (a.muon) Vec8<TM>::load_nt(M + (long long)i * a.cols + j, m[it]);
      }
    }
#pragma unroll
    for (int it = 0; it < NC; ++it) {
      if (!ok[it]) continue;
      const int c = tid + 256 * it;
      const int i = wi * RT + c / (CT / 8), j = wj * CT + (c % (CT / 8)) * 8;
      float u[8];
      if (a.muon) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float ge = Vec8<TM>::round(g[it][e]);             // G.to(M.dtype)
          float me = Vec8<TM>::round(m[it][e] * a.mu);            // M *= mu
          me = Vec8<TM>::round(me + ge);                          // M += G
          m[it][e] = me;
          float ue = me;
          if (a.nesterov) ue = Vec8<TM>::round(Vec8<TM>::round(me * a.mu) + ge);  // U = M*mu; U += G
          u[e] = Vec8<TW>::round(ue);                             // U.to(bf16)
        }
        Vec8<TM>::store_nt(M + (long long)i * a.cols + j, m[it]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = Vec8<TW>::round(g[it][e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += u[e] * u[e];
      Vec8<TW>::store(W + (long long)i * a.ldw + j, u);
    }
    if (!a.partials) return;   // (uniform over the grid)
    const float s = block_sum(ss, red);
    if (tid == 0) a.partials[(long long)b * gridDim.x + blockIdx.x] = s;
    return;
  }
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int c = tid + 256 * it;        // chunk id within tile: 64 rows x 8 chunks
    const int r = c >> 3, cc = (c & 7) * 8;
    const int i = ti * TS + r, j = tj * TS + cc;
    float u[8];
    const bool ok = i < a.rows && j < a.cols;  // cols is a multiple of 8
    if (ok) {
      float g[8];
      Vec8<TG>::load_nt(G + (long long)i * a.ld + j, g);
      if (a.muon) {
        float m[8];
        Vec8<TM>::load_nt(M + (long long)i * a.cols + j, m);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float ge = Vec8<TM>::round(g[e]);                 // G.to(M.dtype)
          float me = Vec8<TM>::round(m[e] * a.mu);                // M *= mu
          me = Vec8<TM>::round(me + ge);                          // M += G
          m[e] = me;
          float ue = me;
          if (a.nesterov) ue = Vec8<TM>::round(Vec8<TM>::round(me * a.mu) + ge);  // U = M*mu; U += G
          u[e] = Vec8<TW>::round(ue);                             // U.to(bf16)
        }
        Vec8<TM>::store_nt(M + (long long)i * a.cols + j, m);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = Vec8<TW>::round(g[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += u[e] * u[e];
      if (!TALL) Vec8<TW>::store(W + (long long)i * a.ldw + j, u);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) u[e] = 0.f;
    }
    if (TALL) {
#pragma unroll
      for (int e = 0; e < 8; ++e) tile[cc + e][r] = u[e];  // tile[source col][source row]
    }
  }
  if (TALL) {
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int c = tid + 256 * it;
      const int p = c >> 3, qq = (c & 7) * 8;   // wide row p = source col, wide cols = source rows
      const int wi = tj * TS + p, wj = ti * TS + qq;
      if (wi < mw && wj < nw) {                 // rows is a multiple of 8
        float u[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = tile[p][qq + e];
        Vec8<TW>::store(W + (long long)wi * a.ldw + wj, u);
      }
    }
  }
  if (!a.partials) return;   // (uniform over the grid)
  const float s = block_sum(ss, red);
  if (tid == 0) a.partials[(long long)b * gridDim.x + blockIdx.x] = s;
}

// ---------------------------------------------------------------------------------------
// norm_finish: divisor[b] = round(round(sqrt(sum)) + eps)   (bf16 working dtype)
//              divisor[b] = sqrt(sum) + eps                 (f32 working dtype)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void norm_finish_kernel(const float* partials, int n, float eps, int bf16_mode,
                                                          float* divisor) {
  __shared__ double red[256];
  const float* p = partials + (long long)blockIdx.x * n;
  double s = 0.0;
  for (int i = threadIdx.x; i < n; i += 256) s += (double)p[i];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    float nrm = sqrtf((float)red[0]);
    float d;
    if (bf16_mode) d = rbf(rbf(nrm) + eps);
    else d = nrm + eps;
    divisor[blockIdx.x] = d;
  }
}

// x / d for a divisor shared by many elements: with rd = RN(1 / d), one residual step on the estimate x * rd gives
// the correctly rounded quotient (three fused operations instead of the dozen of a full division; the pass is
// otherwise bound by its arithmetic).  |x| <= d here (d is the matrix's Frobenius norm plus eps), so nothing
// overflows; a divisor whose reciprocal is zero or not finite takes the plain division (the caller's branch).
__device__ __forceinline__ float div_by(float x, float d, float rd) {
  const float q = x * rd;
  const float rem = __builtin_fmaf(-q, d, x);
  return __builtin_fmaf(rem, rd, q);
}

// The divisor of matrix b from its partial sums of squares: the same fixed-order fp64 sum and the same roundings as
// norm_finish_kernel, so every workgroup of the matrix arrives at the same bits.
__device__ __forceinline__ float divisor_of(const float* partials, int n, float eps, int bf16_mode, double* red) {
  double s = 0.0;
  for (int i = threadIdx.x; i < n; i += 256) s += (double)partials[i];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  const float nrm = sqrtf((float)red[0]);
  return bf16_mode ? rbf(rbf(nrm) + eps) : nrm + eps;
}

// `partials` != null: the divisor is formed here from the matrix's partial sums (n per matrix) instead of being
// read from `divisor` -- one launch less in front of every normalisation.
template <typename TW>
__global__ __launch_bounds__(256) void normalize_kernel(TW* W, long long per_matrix, const float* divisor,
                                                        const float* partials, int n, float eps, int bf16_mode) {
  const int b = blockIdx.y;
  __shared__ double red[256];
  const float d = partials ? divisor_of(partials + (long long)b * n, n, eps, bf16_mode, red) : divisor[b];
  const float rd = 1.f / d;
  const bool fast = __builtin_isfinite(rd) && rd != 0.f;   // (the same for the whole matrix)
  TW* p = W + (long long)b * per_matrix;
  // four 16-byte chunks per thread and trip, all requested before the first is used
  for (long long i0 = (long long)blockIdx.x * 8192; i0 < per_matrix; i0 += (long long)gridDim.x * 8192) {
    float v[4][8];
    bool ok[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const long long i = i0 + (q * 256 + threadIdx.x) * 8;
      ok[q] = i < per_matrix;
      if (ok[q]) Vec8<TW>::load(p + i, v[q]);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (!ok[q]) continue;
      const long long i = i0 + (q * 256 + threadIdx.x) * 8;
      if (fast) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[q][e] = div_by(v[q][e], d, rd);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[q][e] = v[q][e] / d;
      }
      Vec8<TW>::store(p + i, v[q]);
    }
  }
}

// ---------------------------------------------------------------------------------------
// unstage
// ---------------------------------------------------------------------------------------
template <typename TX, typename TW>
struct UnstageArgs {
  DaPtrTable x;       // destinations, one pointer per matrix (rows x cols, row-major, pitch ld)
  const TW* wide;     // [batch][mw][ldw], columns < nw used
  int rows, cols, ld, ldw;
  float decay;        // 1 - lr * weight_decay
  float step;         // adjusted learning rate
  int muon;           // 1: X <- X*decay - wide*step ; 0: X <- wide
  int use_wtab;       // 1: source b is wtab.p[b] (rows x cols contiguous); never with TALL
  DaPtrTable wtab;
  const int* poison;  // optional device word: non-zero = the working matrices are invalid, the result becomes NaN
};

template <typename TX, typename TW, bool TALL>
__global__ __launch_bounds__(256) void unstage_kernel(UnstageArgs<TX, TW> a) {
  __shared__ float tile[TALL ? TS : 1][TS + 1];
  const bool poisoned = a.poison != nullptr && *a.poison != 0;
  const float nan = __builtin_nanf("");
  const int b = blockIdx.y;
  const int tiles_c = (a.cols + TS - 1) / TS;
  const int ti = blockIdx.x / tiles_c, tj = blockIdx.x % tiles_c;
  const int tid = threadIdx.x;
  TX* X = static_cast<TX*>(a.x.p[b]);
  const int mw = TALL ? a.cols : a.rows, nw = TALL ? a.rows : a.cols;
  const TW* W = a.use_wtab ? static_cast<const TW*>(a.wtab.p[b]) : a.wide + (long long)b * mw * a.ldw;

  if (!TALL) {
    const int tiles_cw = (a.cols + CT - 1) / CT;
    const int wi = blockIdx.x / tiles_cw, wj = blockIdx.x % tiles_cw;
    constexpr int NC = RT * CT / 8 / 256;
    float u[NC][8], x[NC][8];
    bool ok[NC];
#pragma unroll
    for (int it = 0; it < NC; ++it) {
      const int c = tid + 256 * it;
      const int i = wi * RT + c / (CT / 8), j = wj * CT + (c % (CT / 8)) * 8;
      ok[it] = i < a.rows && j < a.cols;
      if (ok[it]) {
        Vec8<TW>::load(W + (long long)i * a.ldw + j, u[it]);
        if (a.muon) Vec8<TX>::load_nt(X + (long long)i * a.ld + j, x[it]);
        if (poisoned) {
#pragma unroll
          for (int e = 0; e < 8; ++e) u[it][e] = nan;
        }
      }
    }
#pragma unroll
    for (int it = 0; it < NC; ++it) {
      if (!ok[it]) continue;
      const int c = tid + 256 * it;
      const int i = wi * RT + c / (CT / 8), j = wj * CT + (c % (CT / 8)) * 8;
      TX* xp = X + (long long)i * a.ld + j;
      if (a.muon) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xd = Vec8<TX>::round(x[it][e] * a.decay);    // X *= 1 - lr*wd
          const float t = Vec8<TW>::round(u[it][e] * a.step);      // U * adjusted_lr (U's dtype)
          x[it][e] = xd - t;                                       // X -= U ; rounded by the store
        }
        Vec8<TX>::store_nt(xp, x[it]);
      } else {
        Vec8<TX>::store(xp, u[it]);
      }
    }
    return;
  }
  if (TALL) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int c = tid + 256 * it;
      const int p = c >> 3, qq = (c & 7) * 8;
      const int wi = tj * TS + p, wj = ti * TS + qq;
      float u[8];
      if (wi < mw && wj < nw) Vec8<TW>::load(W + (long long)wi * a.ldw + wj, u);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = 0.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) tile[qq + e][p] = u[e];  // tile[source row][source col]
    }
    __syncthreads();
  }
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int c = tid + 256 * it;
    const int r = c >> 3, cc = (c & 7) * 8;
    const int i = ti * TS + r, j = tj * TS + cc;
    if (i >= a.rows || j >= a.cols) continue;
    float u[8];
    if (TALL) {
#pragma unroll
      for (int e = 0; e < 8; ++e) u[e] = tile[r][cc + e];
    } else {
      Vec8<TW>::load(W + (long long)i * a.ldw + j, u);
    }
    if (poisoned) {
#pragma unroll
      for (int e = 0; e < 8; ++e) u[e] = nan;
    }
    TX* xp = X + (long long)i * a.ld + j;
    if (a.muon) {
      float x[8];
      Vec8<TX>::load_nt(xp, x);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xd = Vec8<TX>::round(x[e] * a.decay);    // X *= 1 - lr*wd
        const float t = Vec8<TW>::round(u[e] * a.step);      // U * adjusted_lr (U's dtype)
        x[e] = xd - t;                                       // X -= U ; rounded by the store
      }
      Vec8<TX>::store_nt(xp, x);
    } else {
      Vec8<TX>::store(xp, u);
    }
  }
}

template <typename TG, typename TM, typename TW>
int stage_launch(const StageArgs<TG, TM, TW>& a, int batch, bool tall, hipStream_t s) {
  const int tiles = tall ? ((a.rows + TS - 1) / TS) * ((a.cols + TS - 1) / TS)
                         : ((a.rows + RT - 1) / RT) * ((a.cols + CT - 1) / CT);
  dim3 grid(tiles, batch);
  if (tall) hipLaunchKernelGGL((stage_wide_kernel<TG, TM, TW, true>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((stage_wide_kernel<TG, TM, TW, false>), grid, dim3(256), 0, s, a);
  return da_launch_status();
}

template <typename TG, typename TM>
int stage_dispatch_w(const DaStage& d, hipStream_t s) {
  if (d.w_dtype == DA_BF16) {
    StageArgs<TG, TM, bf16_t> a{d.g, d.mom, static_cast<bf16_t*>(d.wide), d.partials, d.rows, d.cols, d.ld, d.ldw, d.mu, d.nesterov, d.muon, d.use_wtab, d.wtab};
    return stage_launch(a, d.batch, d.rows > d.cols && !d.use_wtab, s);
  }
  StageArgs<TG, TM, float> a{d.g, d.mom, static_cast<float*>(d.wide), d.partials, d.rows, d.cols, d.ld, d.ldw, d.mu, d.nesterov, d.muon, d.use_wtab, d.wtab};
  return stage_launch(a, d.batch, d.rows > d.cols && !d.use_wtab, s);
}

template <typename TX, typename TW>
int unstage_launch(const DaUnstage& d, hipStream_t s) {
  UnstageArgs<TX, TW> a{d.x, static_cast<const TW*>(d.wide), d.rows, d.cols, d.ld, d.ldw, d.decay, d.step, d.muon, d.use_wtab, d.wtab, d.poison};
  const bool tall = d.rows > d.cols && !d.use_wtab;
  const int tiles = tall ? ((a.rows + TS - 1) / TS) * ((a.cols + TS - 1) / TS)
                         : ((a.rows + RT - 1) / RT) * ((a.cols + CT - 1) / CT);
  dim3 grid(tiles, d.batch);
  if (tall) hipLaunchKernelGGL((unstage_kernel<TX, TW, true>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((unstage_kernel<TX, TW, false>), grid, dim3(256), 0, s, a);
  return da_launch_status();
}

}  // namespace

// Workgroups (and partial sums of squares) per matrix of da_stage_wide: transposing tiles for a tall source.
int da_stage_tiles(int rows, int cols) {
  return rows > cols ? ((rows + TS - 1) / TS) * ((cols + TS - 1) / TS) : ((rows + RT - 1) / RT) * ((cols + CT - 1) / CT);
}

int da_stage_wide(const DaStage& d, hipStream_t s) {
  if (d.batch <= 0 || d.batch > DA_MAX_PTRS) return DA_ERR_LIMIT;
  if ((d.rows | d.cols | d.ld) & 7) return DA_ERR_ALIGN;
  const int gd = d.g_dtype, md = d.muon ? d.m_dtype : d.g_dtype;
  if (gd == DA_BF16 && md == DA_BF16) return stage_dispatch_w<bf16_t, bf16_t>(d, s);
  if (gd == DA_F32 && md == DA_BF16) return stage_dispatch_w<float, bf16_t>(d, s);
  if (gd == DA_BF16 && md == DA_F32) return stage_dispatch_w<bf16_t, float>(d, s);
  if (gd == DA_F32 && md == DA_F32) return stage_dispatch_w<float, float>(d, s);
  return DA_ERR_DTYPE;
}

int da_norm_finish(const float* partials, int tiles, int batch, float eps, int bf16_mode, float* divisor,
                   hipStream_t s) {
  hipLaunchKernelGGL(norm_finish_kernel, dim3(batch), dim3(256), 0, s, partials, tiles, eps, bf16_mode, divisor);
  return da_launch_status();
}

int da_normalize(void* wide, int w_dtype, long long per_matrix, int batch, const float* divisor, hipStream_t s) {
  return da_normalize_from_partials(wide, w_dtype, per_matrix, batch, divisor, nullptr, 0, 0.f, s);
}

int da_normalize_from_partials(void* wide, int w_dtype, long long per_matrix, int batch, const float* divisor,
                               const float* partials, int tiles, float eps, hipStream_t s) {
  if (per_matrix & 7) return DA_ERR_ALIGN;
  if (!divisor && !partials) return DA_ERR_ARG;
  long long blocks = (per_matrix + 8191) / 8192;
  if (blocks > 2048) blocks = 2048;
  dim3 grid((unsigned)blocks, batch);
  if (w_dtype == DA_BF16)
    hipLaunchKernelGGL(normalize_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<bf16_t*>(wide), per_matrix, divisor,
                       partials, tiles, eps, 1);
  else
    hipLaunchKernelGGL(normalize_kernel<float>, grid, dim3(256), 0, s, static_cast<float*>(wide), per_matrix, divisor,
                       partials, tiles, eps, 0);
  return da_launch_status();
}

namespace {
__global__ __launch_bounds__(64) void upload_ptrs_kernel(DaPtrTable t, void** dst, int n) {
  if ((int)threadIdx.x < n) dst[threadIdx.x] = t.p[threadIdx.x];
}
// every element of the matrices becomes NaN if *flag != 0 (the launch that produced them gave up)
__global__ __launch_bounds__(256) void poison_kernel(DaPtrTable t, long long numel, int f32, const int* flag) {
  if (*flag == 0) return;
  const float nan = __builtin_nanf("");
  void* p = t.p[blockIdx.y];
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < numel; i += (long long)gridDim.x * 256) {
    if (f32) static_cast<float*>(p)[i] = nan;
    else static_cast<bf16_t*>(p)[i] = f2bf(nan);
  }
}
}  // namespace

namespace {
__global__ __launch_bounds__(64) void upload_ptrs_multi_kernel(DaPtrUploads u) {
  const int k = blockIdx.x;
  if ((int)threadIdx.x < u.n[k]) u.dst[k][threadIdx.x] = u.t[k].p[threadIdx.x];
}
__global__ __launch_bounds__(256) void poison_multi_kernel(DaPtrUploads u, DaPoisonShape sh, const int* flag) {
  if (*flag == 0) return;
  const int k = blockIdx.z;
  if ((int)blockIdx.y >= u.n[k]) return;
  const float nan = __builtin_nanf("");
  void* p = u.t[k].p[blockIdx.y];
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < sh.numel[k]; i += (long long)gridDim.x * 256) {
    if (sh.f32) static_cast<float*>(p)[i] = nan;
    else static_cast<bf16_t*>(p)[i] = f2bf(nan);
  }
}
}  // namespace

int da_upload_ptrs_multi(const DaPtrUploads& u, int count, hipStream_t s) {
  if (count < 1 || count > DA_MAX_UPLOADS) return DA_ERR_LIMIT;
  hipLaunchKernelGGL(upload_ptrs_multi_kernel, dim3((unsigned)count), dim3(64), 0, s, u);
  return da_launch_status();
}

int da_poison_multi_if(const DaPtrUploads& u, int count, const DaPoisonShape& sh, const int* flag, hipStream_t s) {
  if (!flag || count < 1 || count > DA_MAX_UPLOADS) return DA_ERR_ARG;
  hipLaunchKernelGGL(poison_multi_kernel, dim3(64, DA_MAX_PTRS, (unsigned)count), dim3(256), 0, s, u, sh, flag);
  return da_launch_status();
}

int da_upload_ptrs(const DaPtrTable& t, void** dst, int n, hipStream_t s) {
  if (!dst || n < 1 || n > DA_MAX_PTRS) return DA_ERR_LIMIT;
  hipLaunchKernelGGL(upload_ptrs_kernel, dim3(1), dim3(64), 0, s, t, dst, n);
  return da_launch_status();
}

int da_poison_if(const DaPtrTable& t, int n, long long numel, int dtype, const int* flag, hipStream_t s) {
  if (!flag || n < 1 || n > DA_MAX_PTRS || numel < 1) return DA_ERR_ARG;
  hipLaunchKernelGGL(poison_kernel, dim3(64, (unsigned)n), dim3(256), 0, s, t, numel, dtype == DA_F32 ? 1 : 0, flag);
  return da_launch_status();
}

int da_unstage(const DaUnstage& d, hipStream_t s) {
  if (d.batch <= 0 || d.batch > DA_MAX_PTRS) return DA_ERR_LIMIT;
  if ((d.rows | d.cols | d.ld) & 7) return DA_ERR_ALIGN;
  if (d.x_dtype == DA_BF16 && d.w_dtype == DA_BF16) return unstage_launch<bf16_t, bf16_t>(d, s);
  if (d.x_dtype == DA_F32 && d.w_dtype == DA_BF16) return unstage_launch<float, bf16_t>(d, s);
  if (d.x_dtype == DA_F32 && d.w_dtype == DA_F32) return unstage_launch<float, float>(d, s);
  if (d.x_dtype == DA_BF16 && d.w_dtype == DA_F32) return unstage_launch<bf16_t, float>(d, s);
  return DA_ERR_DTYPE;
}
