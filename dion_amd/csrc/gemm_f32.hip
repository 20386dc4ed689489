// Batched fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32), full fp32 products and
// accumulation -- the all-fp32 configuration of the Dion step and the fp32 evaluation of
// the Newton-Schulz recurrence.
//
//   C[b] (M x N) = s0 * E[b] + s1 * sum_k Aop[b](i,k) * Bop[b](j,k)
//
// 256 threads (2 x 2 wavefronts) per 128 x 128 tile, 16 k per stage, double buffered
// through LDS.  An fp32 MFMA operand is one scalar per lane, so either operand layout is a
// plain indexed LDS read: k-contiguous tiles are kept [128][16+1], k-strided tiles
// [16][128+4], both conflict-free for the 32-rows-per-half-wave fragment read.
#include "common.h"
#include <type_traits>

namespace {

constexpr int BT = 128;
constexpr int BK = 16;
constexpr int KC_LD = BK + 1;
constexpr int KS_LD = BT + 4;
constexpr int KC_FLOATS = BT * KC_LD;
constexpr int KS_FLOATS = BK * KS_LD;

template <bool KS>
__device__ __forceinline__ void load_global(float4 (&r)[2], const float* __restrict__ base, int ld, int row0, int k0,
                                            int rows, int K, int tid) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + 256 * i;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!KS) {
      const int gr = row0 + (c >> 2), gk = k0 + (c & 3) * 4;
      if (gr < rows && gk < K) v = *reinterpret_cast<const float4*>(base + (long long)gr * ld + gk);
    } else {
      const int gk = k0 + (c >> 5), gr = row0 + (c & 31) * 4;
      if (gk < K && gr < rows) v = *reinterpret_cast<const float4*>(base + (long long)gk * ld + gr);
    }
    r[i] = v;
  }
}

template <bool KS>
__device__ __forceinline__ void store_lds(const float4 (&r)[2], float* lds, int tid) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + 256 * i;
    if (!KS) {
      float* p = lds + (c >> 2) * KC_LD + (c & 3) * 4;
      p[0] = r[i].x; p[1] = r[i].y; p[2] = r[i].z; p[3] = r[i].w;
    } else {
      *reinterpret_cast<float4*>(lds + (c >> 5) * KS_LD + (c & 31) * 4) = r[i];
    }
  }
}

template <bool KS>
__device__ __forceinline__ float read_frag(const float* lds, int r0, int ks, int lane) {
  const int row = r0 + (lane & 31), k = ks * 2 + (lane >> 5);
  return KS ? lds[k * KS_LD + row] : lds[row * KC_LD + k];
}

// CBF: C and E are bf16 (fp32 factors updating bf16 weights): the addend is scaled and rounded in C's dtype
// first, as an in-place  X.mul_(s0); X.add_(fp32 update)  on a bf16 tensor does, and the sum is rounded once
// at the store.
template <bool A_KS, bool B_KS, bool SYM, bool CBF>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmDesc d) {
  constexpr int A_FL = A_KS ? KS_FLOATS : KC_FLOATS;
  constexpr int B_FL = B_KS ? KS_FLOATS : KC_FLOATS;
  constexpr int STAGE = A_FL + B_FL;
  __shared__ __attribute__((aligned(16))) float lds[2 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (d.M + BT - 1) / BT, tiles_n = (d.N + BT - 1) / BT;
  const int per_batch = SYM ? tiles_m * (tiles_m + 1) / 2 : tiles_m * tiles_n;
  const int b = blockIdx.x / per_batch;
  int t = blockIdx.x - b * per_batch;
  int ti, tj;
  if (SYM) {
    ti = 0;
    int len = tiles_m;
    while (t >= len) { t -= len; ++ti; --len; }
    tj = ti + t;
  } else {
    ti = t / tiles_n;
    tj = t - ti * tiles_n;
  }
  const int m0 = ti * BT, n0 = tj * BT;
  const float* A = d.Atab ? static_cast<const float*>(d.Atab[b]) : static_cast<const float*>(d.A) + (long long)b * d.sA;
  const float* B = d.Btab ? static_cast<const float*>(d.Btab[b]) : static_cast<const float*>(d.B) + (long long)b * d.sB;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  float4 ra[2], rb[2];
  const int KT = (d.K + BK - 1) / BK;
  load_global<A_KS>(ra, A, d.lda, m0, 0, d.M, d.K, tid);
  load_global<B_KS>(rb, B, d.ldb, n0, 0, d.N, d.K, tid);
  store_lds<A_KS>(ra, lds, tid);
  store_lds<B_KS>(rb, lds + A_FL, tid);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const float* sa = lds + (kt & 1) * STAGE;
    const float* sb = sa + A_FL;
    const bool more = kt + 1 < KT;
    if (more) {
      load_global<A_KS>(ra, A, d.lda, m0, (kt + 1) * BK, d.M, d.K, tid);
      load_global<B_KS>(rb, B, d.ldb, n0, (kt + 1) * BK, d.N, d.K, tid);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
      float af[2], bfv[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = read_frag<A_KS>(sa, wm * 64 + i * 32, ks, lane);
#pragma unroll
      for (int j = 0; j < 2; ++j) bfv[j] = read_frag<B_KS>(sb, wn * 64 + j * 32, ks, lane);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bfv[j], af[i], acc[i][j], 0, 0, 0);
    }
    if (more) {
      float* na = lds + ((kt + 1) & 1) * STAGE;
      store_lds<A_KS>(ra, na, tid);
      store_lds<B_KS>(rb, na + A_FL, tid);
    }
    __syncthreads();
  }

  const bool mirror = SYM && (ti != tj);
  const bool has_e = d.epilogue == DA_EPI_AXPBY;
  typedef typename std::conditional<CBF, bf16_t, float>::type TC;
  TC* const Cbase = d.Ctab ? static_cast<TC*>(d.Ctab[b]) : static_cast<TC*>(d.C) + (long long)b * d.sC;
  const TC* const Ebase = !has_e ? nullptr
                          : d.Etab ? static_cast<const TC*>(d.Etab[b])
                                   : static_cast<const TC*>(d.E) + (long long)b * d.sE;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = m0 + wm * 64 + i * 32 + (lane & 31);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const int n = n0 + wn * 64 + j * 32 + vq * 8 + (lane >> 5) * 4;
        if (m >= d.M || n >= d.N) continue;
        TC* Cp = Cbase + (long long)m * d.ldc + n;
        float o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = d.s1 * acc[i][j][vq * 4 + q];
        if constexpr (CBF) {
          if (has_e) {
            const uint2 ev = *reinterpret_cast<const uint2*>(Ebase + (long long)m * d.lde + n);
            const float e[4] = {__builtin_bit_cast(float, ev.x << 16), __builtin_bit_cast(float, ev.x & 0xffff0000u),
                                __builtin_bit_cast(float, ev.y << 16), __builtin_bit_cast(float, ev.y & 0xffff0000u)};
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = rbf(d.s0 * e[q]) + o[q];
          }
          uint2 w;
          w.x = (uint32_t)f2bf(o[0]) | ((uint32_t)f2bf(o[1]) << 16);
          w.y = (uint32_t)f2bf(o[2]) | ((uint32_t)f2bf(o[3]) << 16);
          *reinterpret_cast<uint2*>(Cp) = w;
        } else {
          if (has_e) {
            const float4 ev = *reinterpret_cast<const float4*>(Ebase + (long long)m * d.lde + n);
            o[0] = d.s0 * ev.x + o[0]; o[1] = d.s0 * ev.y + o[1];
            o[2] = d.s0 * ev.z + o[2]; o[3] = d.s0 * ev.w + o[3];
          }
          *reinterpret_cast<float4*>(Cp) = make_float4(o[0], o[1], o[2], o[3]);
        }
        if (mirror) {
          TC* Ct = Cbase + (long long)n * d.ldc + m;
#pragma unroll
          for (int q = 0; q < 4; ++q) st_from_float<TC>(Ct + (long long)q * d.ldc, o[q]);
        }
      }
    }
  }
}

template <bool A_KS, bool B_KS, bool SYM>
int launch(const GemmDesc& d, hipStream_t stream) {
  const bool cbf = d.c_dtype == DA_BF16;
  const int tiles_m = (d.M + BT - 1) / BT, tiles_n = (d.N + BT - 1) / BT;
  const long long per_batch = SYM ? (long long)tiles_m * (tiles_m + 1) / 2 : (long long)tiles_m * tiles_n;
  const long long blocks = per_batch * d.batch;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return DA_ERR_LIMIT;
  if (cbf) hipLaunchKernelGGL((gemm_f32_kernel<A_KS, B_KS, SYM, true>), dim3((unsigned)blocks), dim3(256), 0, stream, d);
  else hipLaunchKernelGGL((gemm_f32_kernel<A_KS, B_KS, SYM, false>), dim3((unsigned)blocks), dim3(256), 0, stream, d);
  return da_launch_status();
}

}  // namespace

// Alignment contract: K, N, leading dimensions and batch strides multiples of 4 elements,
// M too when A is k-strided; pointers 16-byte aligned.  C and E are fp32, or bf16 (rounded at the store).
int da_gemm_f32(const GemmDesc& d, hipStream_t stream) {
  if ((!d.A && !d.Atab) || (!d.B && !d.Btab) || (!d.C && !d.Ctab) || d.M <= 0 || d.N <= 0 || d.K <= 0 || d.batch <= 0) return DA_ERR_ARG;
  if (d.epilogue == DA_EPI_AXPBY && !d.E && !d.Etab) return DA_ERR_ARG;
  if (d.c_dtype != DA_F32 && d.c_dtype != DA_BF16) return DA_ERR_DTYPE;
  if ((d.K | d.N | d.lda | d.ldb | d.ldc) & 3) return DA_ERR_ALIGN;
  if ((d.sA | d.sB | d.sC) & 3) return DA_ERR_ALIGN;
  if ((d.E || d.Etab) && ((d.lde & 3) || (d.sE & 3))) return DA_ERR_ALIGN;
  if (d.a_kstrided && (d.M & 3)) return DA_ERR_ALIGN;
  if (((uintptr_t)d.A | (uintptr_t)d.B | (uintptr_t)d.C | (uintptr_t)d.E) & 15) return DA_ERR_ALIGN;
  if (d.symmetric) {
    if (d.M != d.N || d.a_kstrided || d.b_kstrided) return DA_ERR_ARG;
    return launch<false, false, true>(d, stream);
  }
  if (!d.a_kstrided && !d.b_kstrided) return launch<false, false, false>(d, stream);
  if (!d.a_kstrided && d.b_kstrided) return launch<false, true, false>(d, stream);
  if (d.a_kstrided && !d.b_kstrided) return launch<true, false, false>(d, stream);
  return launch<true, true, false>(d, stream);
}
