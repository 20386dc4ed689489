// Lion and AdamW for the parameter groups that are not matrices (embeddings, lm_head, norms,
// biases): one fused multi-tensor pass each, in place, HBM-bound.  Replaces the reference's
// lion_update_foreach / adamw_update_foreach (dion/scalar_opts.py:152-187, 89-149), whose every
// tensor op is a separate pass over memory; the rounding points of those ops (each result is
// rounded to the dtype of the tensor that holds it) are reproduced in registers.
//
//   Lion :  g = r_M(G);  U = sign(r_M(lerp(M, g, r_M(1-b1))));  M <- r_M(lerp(M, g, r_M(1-b2)));
//           X <- r_X(X * (1 - lr wd));  X <- r_X(X - r_M(U * lr))
//   AdamW:  g = r_M(G);  M <- r_M(lerp(M, g, r_M(1-b1)));  V <- r_V(lerp(V, r_V(r_M(g g)), r_V(1-b2)));
//           den = r_V(r_V(r_V(sqrt V) / sqrt(1-b2^t)) + eps);  X <- r_X(X * (1 - lr wd));
//           X <- r_X(X - r_D(r_D(M / den) * lr / (1-b1^t)))          (D = the wider of M's and V's dtype)
//
// Tensors of one call share their dtypes; each has its own length.  A tensor whose pointers are
// all 16-byte aligned moves as 8-element vectors (plus a scalar tail), any other element by element.
#include "../../include/dion_amd.h"
#include "common.h"
#include "prof.h"

namespace {

constexpr int MAX_TENSORS = 48;   // per launch: the table travels as a kernel argument

struct ScalarTable {
  void* x[MAX_TENSORS];
  const void* g[MAX_TENSORS];
  void* m[MAX_TENSORS];
  void* v[MAX_TENSORS];
  long long n[MAX_TENSORS];
  int first_block[MAX_TENSORS + 1]; // tensor i owns blocks first_block[i] .. first_block[i+1]-1
  unsigned char vec[MAX_TENSORS];   // 1: every pointer of the tensor is 16-byte aligned
  int count;
};

constexpr int BLOCK_ELEMS = 256 * 8 * 4;   // elements per workgroup: four 8-element vectors per lane

struct ScalarArgs {
  float w1, w2;        // 1 - beta1, 1 - beta2 (lerp weights)
  float decay;         // 1 - lr * weight_decay
  float lr;            // Lion: lr;  AdamW: lr / (1 - beta1^step)
  float bc2_sqrt;      // AdamW: sqrt(1 - beta2^step)
  float eps;           // AdamW
  int x_dtype, g_dtype, m_dtype, v_dtype;
};

__device__ __forceinline__ float rnd(float x, int dtype) { return dtype == DA_BF16 ? rbf(x) : x; }

// torch.lerp with a 0-dim tensor weight: the weight is first cast to the dtype of the tensors (so in
// bf16 1 - 0.95 becomes 0.050048828125), then start + w (end - start) for |w| < 0.5, else
// end - (end - start)(1 - w); one rounding of the fused multiply-add in fp32, then the store's rounding
__device__ __forceinline__ float lerp_f(float s, float e, float w_in, int dtype) {
  const float w = rnd(w_in, dtype);
  const float d = e - s;
  return fabsf(w) < 0.5f ? fmaf(w, d, s) : fmaf(-(1.0f - w), d, e);
}

__device__ __forceinline__ float ld1(const void* p, int dtype, long long i) {
  return dtype == DA_BF16 ? bf2f(static_cast<const bf16_t*>(p)[i]) : static_cast<const float*>(p)[i];
}
__device__ __forceinline__ void st1(void* p, int dtype, long long i, float v) {
  if (dtype == DA_BF16) static_cast<bf16_t*>(p)[i] = f2bf(v);
  else static_cast<float*>(p)[i] = v;
}
// 8 elements per lane with non-temporal hints: every operand is touched once per step
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void ld8(const void* p, int dtype, long long i, float (&v)[8]) {
  if (dtype == DA_BF16) {
    const u32x4_t w = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(static_cast<const bf16_t*>(p) + i));
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v[2 * q] = __builtin_bit_cast(float, w[q] << 16);
      v[2 * q + 1] = __builtin_bit_cast(float, w[q] & 0xffff0000u);
    }
  } else {
    const u32x4_t* src = reinterpret_cast<const u32x4_t*>(static_cast<const float*>(p) + i);
    const u32x4_t a = __builtin_nontemporal_load(src), b = __builtin_nontemporal_load(src + 1);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned ua = a[q], ub = b[q];   // (bit_cast applied directly to a vector element reads element 0)
      v[q] = __builtin_bit_cast(float, ua);
      v[4 + q] = __builtin_bit_cast(float, ub);
    }
  }
}
__device__ __forceinline__ void st8(void* p, int dtype, long long i, const float (&v)[8]) {
  if (dtype == DA_BF16) {
    u32x4_t w;
#pragma unroll
    for (int q = 0; q < 4; ++q) w[q] = (uint32_t)f2bf(v[2 * q]) | ((uint32_t)f2bf(v[2 * q + 1]) << 16);
    __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t*>(static_cast<bf16_t*>(p) + i));
  } else {
    u32x4_t a, b;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      a[q] = __builtin_bit_cast(unsigned, v[q]);
      b[q] = __builtin_bit_cast(unsigned, v[4 + q]);
    }
    u32x4_t* dst = reinterpret_cast<u32x4_t*>(static_cast<float*>(p) + i);
    __builtin_nontemporal_store(a, dst);
    __builtin_nontemporal_store(b, dst + 1);
  }
}

__device__ __forceinline__ void lion_one(float& x, float gin, float& m, const ScalarArgs& a) {
  const float g = rnd(gin, a.m_dtype);
  const float u0 = rnd(lerp_f(m, g, a.w1, a.m_dtype), a.m_dtype);
  const float u = u0 > 0.f ? 1.f : (u0 < 0.f ? -1.f : u0);   // sign keeps 0 and NaN
  m = rnd(lerp_f(m, g, a.w2, a.m_dtype), a.m_dtype);
  const float xd = rnd(x * a.decay, a.x_dtype);
  const float step = rnd(u * a.lr, a.m_dtype);
  x = xd - step;   // rounded by the store
}

__device__ __forceinline__ void adamw_one(float& x, float gin, float& m, float& v, const ScalarArgs& a) {
  const int d_dtype = (a.m_dtype == DA_F32 || a.v_dtype == DA_F32) ? DA_F32 : DA_BF16;
  const float g = rnd(gin, a.m_dtype);
  m = rnd(lerp_f(m, g, a.w1, a.m_dtype), a.m_dtype);
  const float g2 = rnd(rnd(g * g, a.m_dtype), a.v_dtype);
  v = rnd(lerp_f(v, g2, a.w2, a.v_dtype), a.v_dtype);
  float den = rnd(sqrtf(v), a.v_dtype);
  den = rnd(den / a.bc2_sqrt, a.v_dtype);
  den = rnd(den + a.eps, a.v_dtype);
  const float xd = rnd(x * a.decay, a.x_dtype);
  float q = rnd(m / den, d_dtype);
  q = rnd(q * a.lr, d_dtype);
  x = xd - q;      // rounded by the store
}

// DT: dtype code shared by X, G, M and V when known at compile time (the common cases: all bf16, all fp32), so that the
// per-element rounding and load / store forms carry no branches; -1: the codes of `ain` decide at run time.
template <bool ADAMW, int DT>
__global__ __launch_bounds__(256) void scalar_opt_kernel(ScalarTable t, ScalarArgs ain) {
  ScalarArgs a = ain;
  if (DT >= 0) { a.x_dtype = DT; a.g_dtype = DT; a.m_dtype = DT; a.v_dtype = DT; }
  // which tensor this workgroup works on: bisection over the block ranges
  int lo = 0, hi = t.count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int)blockIdx.x >= t.first_block[mid]) lo = mid; else hi = mid - 1;
  }
  const int b = lo;
  void* X = t.x[b];
  const void* G = t.g[b];
  void* M = t.m[b];
  void* V = ADAMW ? t.v[b] : nullptr;
  const long long n = t.n[b];
  const long long nvec = t.vec[b] ? n / 8 * 8 : 0;
  const long long begin = (long long)((int)blockIdx.x - t.first_block[b]) * BLOCK_ELEMS;
  const long long end = begin + BLOCK_ELEMS < n ? begin + BLOCK_ELEMS : n;
  const long long vend = end < nvec ? end : nvec;
  if (vend - begin == BLOCK_ELEMS) {
    // a whole block: the four vectors of a lane are requested before the first is used
    constexpr int NV = BLOCK_ELEMS / (256 * 8);
    float x[NV][8], g[NV][8], m[NV][8], v[NV][8];
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const long long i = begin + (q * 256 + threadIdx.x) * 8;
      ld8(X, a.x_dtype, i, x[q]);
      ld8(G, a.g_dtype, i, g[q]);
      ld8(M, a.m_dtype, i, m[q]);
      if (ADAMW) ld8(V, a.v_dtype, i, v[q]);
    }
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const long long i = begin + (q * 256 + threadIdx.x) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (ADAMW) adamw_one(x[q][e], g[q][e], m[q][e], v[q][e], a);
        else lion_one(x[q][e], g[q][e], m[q][e], a);
      }
      st8(X, a.x_dtype, i, x[q]);
      st8(M, a.m_dtype, i, m[q]);
      if (ADAMW) st8(V, a.v_dtype, i, v[q]);
    }
    return;
  }
  for (long long i = begin + threadIdx.x * 8; i < vend; i += 256 * 8) {
    float x[8], g[8], m[8], v[8];
    ld8(X, a.x_dtype, i, x);
    ld8(G, a.g_dtype, i, g);
    ld8(M, a.m_dtype, i, m);
    if (ADAMW) ld8(V, a.v_dtype, i, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (ADAMW) adamw_one(x[e], g[e], m[e], v[e], a);
      else lion_one(x[e], g[e], m[e], a);
    }
    st8(X, a.x_dtype, i, x);
    st8(M, a.m_dtype, i, m);
    if (ADAMW) st8(V, a.v_dtype, i, v);
  }
  // unaligned tensors entirely, aligned ones for their last n % 8 elements
  for (long long i = (begin > nvec ? begin : nvec) + threadIdx.x; i < end; i += 256) {
    float x = ld1(X, a.x_dtype, i), m = ld1(M, a.m_dtype, i), v = ADAMW ? ld1(V, a.v_dtype, i) : 0.f;
    const float g = ld1(G, a.g_dtype, i);
    if (ADAMW) adamw_one(x, g, m, v, a);
    else lion_one(x, g, m, a);
    st1(X, a.x_dtype, i, x);
    st1(M, a.m_dtype, i, m);
    if (ADAMW) st1(V, a.v_dtype, i, v);
  }
}

inline bool dtype_ok(int d) { return d == DA_BF16 || d == DA_F32; }
inline size_t esize(int d) { return d == DA_BF16 ? 2 : 4; }

int run(bool adamw, void* const* X, const void* const* G, void* const* M, void* const* V, const long long* numel,
        int count, const ScalarArgs& a, hipStream_t s) {
  if (!X || !G || !M || (adamw && !V) || !numel || count <= 0) return DA_ERR_ARG;
  if (!dtype_ok(a.x_dtype) || !dtype_ok(a.g_dtype) || !dtype_ok(a.m_dtype) || (adamw && !dtype_ok(a.v_dtype)))
    return DA_ERR_DTYPE;
  for (int i = 0; i < count; ++i) {
    if (numel[i] < 0) return DA_ERR_ARG;
    if (numel[i] == 0) continue;   // empty tensors may come without storage
    if (!X[i] || !G[i] || !M[i] || (adamw && !V[i])) return DA_ERR_ARG;
    // element alignment is the least a tensor of that dtype has
    if (((uintptr_t)X[i] % esize(a.x_dtype)) || ((uintptr_t)G[i] % esize(a.g_dtype)) ||
        ((uintptr_t)M[i] % esize(a.m_dtype)) || (adamw && ((uintptr_t)V[i] % esize(a.v_dtype))))
      return DA_ERR_ALIGN;
  }
  for (int i0 = 0; i0 < count; i0 += MAX_TENSORS) {
    const int c = count - i0 < MAX_TENSORS ? count - i0 : MAX_TENSORS;
    ScalarTable t{};
    long long blocks = 0;
    double bytes = 0.0;
    int k = 0;
    for (int i = 0; i < c; ++i) {
      if (numel[i0 + i] == 0) continue;
      t.x[k] = X[i0 + i];
      t.g[k] = G[i0 + i];
      t.m[k] = M[i0 + i];
      t.v[k] = adamw ? V[i0 + i] : nullptr;
      t.n[k] = numel[i0 + i];
      const uintptr_t all = (uintptr_t)t.x[k] | (uintptr_t)t.g[k] | (uintptr_t)t.m[k] | (uintptr_t)t.v[k];
      t.vec[k] = (all & 15) == 0;
      t.first_block[k] = (int)blocks;
      blocks += (t.n[k] + BLOCK_ELEMS - 1) / BLOCK_ELEMS;
      if (blocks > 0x7fffffffLL) return DA_ERR_LIMIT;
      // algorithmic bytes: read X, G, M (, V); write X, M (, V)
      bytes += (double)t.n[k] * (2.0 * esize(a.x_dtype) + esize(a.g_dtype) + 2.0 * esize(a.m_dtype) +
                                 (adamw ? 2.0 * esize(a.v_dtype) : 0.0));
      ++k;
    }
    if (k == 0) continue;
    t.count = k;
    for (int i = k; i <= MAX_TENSORS; ++i) t.first_block[i] = (int)blocks;
    DaProfScope prof(DA_PROF_SCALAR_OPT, bytes, s);
    const bool same = a.g_dtype == a.x_dtype && a.m_dtype == a.x_dtype && (!adamw || a.v_dtype == a.x_dtype);
    const int dt = same ? a.x_dtype : -1;
    const dim3 grid((unsigned)blocks), block(256);
#define DA_SCALAR_LAUNCH(AD, DT) hipLaunchKernelGGL((scalar_opt_kernel<AD, DT>), grid, block, 0, s, t, a)
    if (adamw) {
      if (dt == DA_BF16) DA_SCALAR_LAUNCH(true, DA_BF16);
      else if (dt == DA_F32) DA_SCALAR_LAUNCH(true, DA_F32);
      else DA_SCALAR_LAUNCH(true, -1);
    } else {
      if (dt == DA_BF16) DA_SCALAR_LAUNCH(false, DA_BF16);
      else if (dt == DA_F32) DA_SCALAR_LAUNCH(false, DA_F32);
      else DA_SCALAR_LAUNCH(false, -1);
    }
#undef DA_SCALAR_LAUNCH
    const int rc = da_launch_status();
    if (rc) return rc;
  }
  return DA_OK;
}

}  // namespace

extern "C" {

int dion_amd_lion_step(void* const* X, const void* const* G, void* const* M, const long long* numel, int count,
                       int x_dtype, int g_dtype, int m_dtype, float lr, float one_minus_beta1,
                       float one_minus_beta2, float decay, void* stream) {
  ScalarArgs a{};
  a.w1 = one_minus_beta1; a.w2 = one_minus_beta2; a.decay = decay; a.lr = lr;
  a.x_dtype = x_dtype; a.g_dtype = g_dtype; a.m_dtype = m_dtype; a.v_dtype = m_dtype;
  return run(false, X, G, M, nullptr, numel, count, a, static_cast<hipStream_t>(stream));
}

int dion_amd_adamw_step(void* const* X, const void* const* G, void* const* M, void* const* V,
                        const long long* numel, int count, int x_dtype, int g_dtype, int m_dtype, int v_dtype,
                        float adjusted_lr, float one_minus_beta1, float one_minus_beta2, float decay,
                        float bias_correction2_sqrt, float epsilon, void* stream) {
  ScalarArgs a{};
  a.w1 = one_minus_beta1; a.w2 = one_minus_beta2; a.decay = decay; a.lr = adjusted_lr;
  a.bc2_sqrt = bias_correction2_sqrt; a.eps = epsilon;
  a.x_dtype = x_dtype; a.g_dtype = g_dtype; a.m_dtype = m_dtype; a.v_dtype = v_dtype;
  return run(true, X, G, M, V, numel, count, a, static_cast<hipStream_t>(stream));
}

}  // extern "C"
