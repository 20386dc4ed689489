// Shared declarations for the gfx950 kernels of the Muon / Dion optimizer step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <atomic>

// ---- error codes of the C ABI (0 ok, <0 bad argument, >0 hipError_t) -------------
#define DA_OK 0
#define DA_ERR_ARG (-1)        // null pointer / non-positive size
#define DA_ERR_ALIGN (-2)      // a dimension or leading dimension breaks an alignment rule
#define DA_ERR_WORKSPACE (-3)  // workspace too small
#define DA_ERR_DTYPE (-4)      // unsupported dtype code
#define DA_ERR_LIMIT (-5)      // size beyond a documented maximum

// ---- dtype codes -------------------------------------------------------------------
#define DA_BF16 0
#define DA_F32 1
#define DA_F64 2

typedef uint16_t bf16_t;  // storage type; arithmetic always goes through float

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef double f64x4_t __attribute__((ext_vector_type(4)));

#define DA_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// Round-to-nearest-even float -> bf16 storage bits, and back.
__device__ __forceinline__ bf16_t f2bf(float f) {
  __bf16 h = (__bf16)f;
  return __builtin_bit_cast(bf16_t, h);
}
__device__ __forceinline__ float bf2f(bf16_t h) {
  return __builtin_bit_cast(float, ((uint32_t)h) << 16);
}
// Round a float to bf16 precision and keep it as float (one rounding point of the
// reference's op-by-op bf16 arithmetic).
__device__ __forceinline__ float rbf(float f) { return bf2f(f2bf(f)); }

template <typename T> __device__ __forceinline__ float ld_as_float(const T* p);
template <> __device__ __forceinline__ float ld_as_float<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ld_as_float<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void st_from_float(T* p, float v);
template <> __device__ __forceinline__ void st_from_float<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void st_from_float<float>(float* p, float v) { *p = v; }

#define DA_HIP_CHECK(expr)                       \
  do {                                           \
    hipError_t e__ = (expr);                     \
    if (e__ != hipSuccess) return (int)e__;      \
  } while (0)

static inline int da_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DA_OK : (int)e;
}

// Compute units of the current device (persistent kernels size their grids with it).  Callers may be on several
// host threads at once: the cache entries are atomics (racing first calls store the same value).
static inline int da_cu_count() {
  static std::atomic<int> cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cache[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cache[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// One-time set-up of a kernel (its dynamic shared memory limit) per device.  The set-up call is idempotent, so two
// host threads that race on the first launch may both make it; the flag word itself is an atomic with one bit per
// device, set only after the call succeeded.
struct DaOncePerDevice {
  std::atomic<unsigned long long> done{0};
  template <typename F>
  int run(F&& setup) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    const unsigned long long bit = 1ull << dev;
    if (done.load(std::memory_order_acquire) & bit) return DA_OK;
    const int rc = setup();
    if (rc == DA_OK) done.fetch_or(bit, std::memory_order_release);
    return rc;
  }
};

// ---- GEMM descriptor shared by the bf16 / f32 / f64 kernels -------------------------
// C[b] (M x N) = epilogue( sum_k Aop[b](i,k) * Bop[b](j,k) ).
// An operand is either "k-contiguous" (stored rows x K, ld = row pitch) or
// "k-strided" (stored K x rows, ld = k pitch).  All pitches / strides in elements.
struct GemmDesc {
  const void* A;
  const void* B;
  void* C;
  const void* E;      // epilogue operand (same shape / layout as C), may be null
  // Optional device arrays of per-matrix base pointers; when set they replace base + b * stride
  // (matrices that live in separate allocations, e.g. the optimizer's momentum buffers).
  const void* const* Atab;
  const void* const* Btab;
  void* const* Ctab;
  const void* const* Etab;
  long long a_off;    // elements added to Atab[b]: a K-slice of operands that are addressed through the table (bf16 kernel)
  long long sA, sB, sC, sE;  // batch strides
  int lda, ldb, ldc, lde;
  int M, N, K;
  int batch;
  int a_kstrided, b_kstrided;
  int symmetric;      // 1: C is symmetric (M == N); compute upper tiles and mirror
  int epilogue;       // DA_EPI_*
  int faithful;       // 1: reproduce every bf16 rounding of the op-by-op reference
  float s0, s1;       // epilogue scalars
  int c_dtype;        // dtype of C / E for the f32 and f64 kernels' mixed outputs
  // Optional per-matrix switch (bf16 kernel): with `gate` set, matrix b is computed only if
  // (gate[b] != 0) == (gate_want != 0); the workgroups of the other matrices return at once.
  const int* gate;
  int gate_want;
  // bf16 kernel, optional.  a_kwrap > 0: A has only a_kwrap columns (a multiple of 64 that divides K; A k-contiguous)
  // and is read again from its first column every a_kwrap steps of k: C = A [B_0; B_1; ...] = sum_i A B_i in one
  // accumulation.  c2_off != 0 (bf16 C, plain store): the part of s1 * acc that the bf16 value stored in C leaves
  // over is rounded to bf16 as well and stored c2_off elements after C -- the result as two bf16 matrices.
  int a_kwrap;
  long long c2_off;
  // bf16 kernel, optional.  k_slices > 1: the sum over k is cut into that many slices of k_slice elements (a multiple
  // of 64; the last one may be shorter) that run as tiles of their own; slice s stores its partial product as
  // matrices s * batch ... s * batch + batch - 1 of C, which therefore holds k_slices * batch matrices sC apart,
  // and the caller adds them in a fixed order.  Plain fp32 store only (no E, no tables, no second output).
  int k_slices, k_slice;
  // bf16 kernel, optional (bf16 result with an epilogue operand, not symmetric, interior tiles).  upd_tab != null:
  // the result C is not stored; it is the update of the matrix upd_tab[b] (upd_dtype, row pitch upd_ld), in place:
  //   W <- r_W( r_W(W * upd_decay) - r_bf16(C * upd_step) )
  // element (i, j) of C updating W[i][j], or W[j][i] when upd_transposed (W is stored N x M).
  void* const* upd_tab;
  int upd_dtype, upd_ld, upd_transposed;
  float upd_decay, upd_step;
  // bf16 only, both operands k-contiguous, not symmetric: run the product with v_mfma_f32_32x32x16_bf16 (16 values of k
  // per instruction instead of 32: another order of the fp32 sums).  Dion's error-feedback and weight-update products
  // use it so that their bits are those of the one-pass kernel (dion_fused.hip), which is built on that instruction.
  int mi32;
};

// Epilogues.  With `faithful` set the rounding points of the reference's separate
// tensor ops are reproduced: t = r_in(acc); t = r_in(s1 * t) (skipped when s1 == 1);
// e = r_c(s0 * E); C = r_c(e + t), where r_in rounds to the GEMM's input dtype (the
// dtype a library matmul would have returned) and r_c to C's dtype.  Otherwise
// C = r_c(s0 * E + s1 * acc) with a single rounding.
#define DA_EPI_STORE 0  // C = s1 * acc
#define DA_EPI_AXPBY 1  // C = s0 * E + s1 * acc; E may alias C (in-place update)

int da_gemm_bf16(const GemmDesc& d, hipStream_t stream);

// Several independent batched bf16 GEMMs of the same form (operand layouts, symmetry, epilogue
// kind and output dtype) in one launch: their tiles share the grid, so a product too small to
// fill the chip runs beside the others instead of after them.
constexpr int DA_MAX_GROUPS = 4;
int da_gemm_bf16_grouped(const GemmDesc* d, int n, hipStream_t stream);
int da_gemm_f32(const GemmDesc& d, hipStream_t stream);
// Tile edge (128 / 256) the bf16 launcher picks for one product, + 1 if its K loop is the direct-to-LDS one.
int da_gemm_bf16_plan(const GemmDesc& d);
// -1 / 0 / 1: whether ragged products may take the direct-to-LDS K loop with edge tiles (see dion_amd_set_option)
void da_gemm_bf16_set_edge_loop(int v);
// Whether da_gemm_bf16_grouped would run every tile of these products in its interior (unchecked) form.
bool da_gemm_bf16_all_interior(const GemmDesc* d, int n);
