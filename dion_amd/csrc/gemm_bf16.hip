// Batched bf16 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate).
//
//   C[b] (M x N) = epilogue( sum_k Aop[b](i,k) * Bop[b](j,k) )
//
// Work decomposition: one 256-thread workgroup (4 wavefronts of 64 lanes, 2 x 2) per
// BT x BT output tile, BT in {128, 256}; each wavefront owns a (BT/2) x (BT/2) sub-tile
// as (BT/64)^2 accumulators of 32 x 32.  The K loop advances 64 elements per stage and
// is double buffered through LDS: while the matrix cores work on stage s, the 16-byte
// global loads of stage s+1 are in flight in registers.
//
// Operand staging in LDS:
//   * k-contiguous operand (rows x K in memory): tile [BT][64] of 16-byte chunks, chunk
//     index XOR-swizzled with (row & 7) so that the 32 rows one ds_read_b128 fragment
//     read touches spread over all banks.
//   * k-strided operand (K x rows in memory, e.g. X in  X' = aX + B X): the tile is kept
//     exactly as it lies in memory, [64][BT + 16], and the fragment is fetched with two
//     ds_read_b64_tr_b16 (the LDS transpose read of CDNA4), which hands each lane the four
//     k-consecutive values of its own column.  No register shuffles, no second copy of X.
//
// The MFMA is issued with the operands swapped (D' = Bfrag x Afrag^T), so that a lane ends
// up with four *column-consecutive* results of one output row: 8-byte epilogue loads and
// stores for row-major C and E.  For a symmetric result only tiles on or above the
// diagonal are computed and every off-diagonal tile is also written transposed.
#include "common.h"

namespace {

constexpr int BK = 64;       // k elements per stage
constexpr int KS_PAD = 16;   // padding (elements) per k-row of a k-strided LDS tile

template <int BT, bool KS>
struct Tile {
  static constexpr int ks_ld = BT + KS_PAD;
  static constexpr int bytes = KS ? BK * ks_ld * 2 : BT * BK * 2;
  static constexpr int chunks = BT / 32;  // 16-byte chunks per thread per stage
};

template <int BT, bool KS>
__device__ __forceinline__ void load_tile_global(uint4 (&r)[BT / 32], const bf16_t* __restrict__ base, int ld,
                                                 int row0, int k0, int rows, int K, int tid) {
#pragma unroll
  for (int i = 0; i < BT / 32; ++i) {
    const int c = tid + 256 * i;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (!KS) {
      const int gr = row0 + (c >> 3);
      const int gk = k0 + (c & 7) * 8;
      if (gr < rows && gk < K) v = *reinterpret_cast<const uint4*>(base + (long long)gr * ld + gk);
    } else {
      constexpr int CPR = BT / 8;  // chunks per k-row
      const int gk = k0 + c / CPR;
      const int gr = row0 + (c % CPR) * 8;
      if (gk < K && gr < rows) v = *reinterpret_cast<const uint4*>(base + (long long)gk * ld + gr);
    }
    r[i] = v;
  }
}

template <int BT, bool KS>
__device__ __forceinline__ void store_tile_lds(const uint4 (&r)[BT / 32], char* lds, int tid) {
#pragma unroll
  for (int i = 0; i < BT / 32; ++i) {
    const int c = tid + 256 * i;
    if (!KS) {
      const int row = c >> 3;
      const int phys = (c & 7) ^ (row & 7);
      *reinterpret_cast<uint4*>(lds + row * 128 + phys * 16) = r[i];
    } else {
      constexpr int CPR = BT / 8;
      const int kr = c / CPR;
      const int mc = c % CPR;
      *reinterpret_cast<uint4*>(lds + (kr * Tile<BT, true>::ks_ld + mc * 8) * 2) = r[i];
    }
  }
}

// Fragment of 32 rows x 16 k for one MFMA: lane l gets row (l & 31), k = 8 * (l >> 5) .. +8.
template <int BT, bool KS>
__device__ __forceinline__ bf16x8_t read_frag(const char* lds, int r0, int ks, int lane) {
  if (!KS) {
    const int row = r0 + (lane & 31);
    const int phys = (ks * 2 + (lane >> 5)) ^ (row & 7);
    const uint4 v = *reinterpret_cast<const uint4*>(lds + row * 128 + phys * 16);
    return __builtin_bit_cast(bf16x8_t, v);
  } else {
    // Per 16-lane group g: rows r0 + 16 * (g & 1) .. +16, k-group g >> 1.  The four lanes
    // 4q .. 4q+3 of a group together supply 16 consecutive rows of k-row q; the transpose
    // read returns to lane i of the group the four k values of row i.
    constexpr int LD = Tile<BT, true>::ks_ld;
    const int g = lane >> 4;
    const int col = r0 + (g & 1) * 16 + (lane & 3) * 4;
    const int kr = ks * 16 + (g >> 1) * 8 + ((lane & 15) >> 2);
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(DA_LDS_PTR(s16x4_t, lds + (kr * LD + col) * 2));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(DA_LDS_PTR(s16x4_t, lds + ((kr + 4) * LD + col) * 2));
    typedef short s16x8_t __attribute__((ext_vector_type(8)));
    const s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, v);
  }
}

struct Epi {
  float s0, s1;
  int mode, faithful, c_f32;
};

// value of C from the accumulator and (optionally) the epilogue operand
__device__ __forceinline__ float epi_value(const Epi& ep, float acc, float e) {
  if (ep.faithful) {
    float t = rbf(acc);
    t = rbf(ep.s1 * t);
    if (ep.mode == DA_EPI_AXPBY) {
      float u = ep.s0 * e;
      if (!ep.c_f32) u = rbf(u);
      t = u + t;
    }
    return t;  // final rounding to C's dtype happens at the store
  }
  return ep.mode == DA_EPI_AXPBY ? ep.s0 * e + ep.s1 * acc : ep.s1 * acc;
}

template <int BT, bool A_KS, bool B_KS, bool SYM>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(GemmDesc d) {
  constexpr int TM = BT / 64;  // 32x32 accumulators per wavefront in each direction
  constexpr int A_BYTES = Tile<BT, A_KS>::bytes;
  constexpr int B_BYTES = Tile<BT, B_KS>::bytes;
  constexpr int STAGE = A_BYTES + B_BYTES;
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which tile ---------------------------------------------------------------
  const int tiles_m = (d.M + BT - 1) / BT;
  const int tiles_n = (d.N + BT - 1) / BT;
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

  const bf16_t* A = d.Atab ? static_cast<const bf16_t*>(d.Atab[b]) : static_cast<const bf16_t*>(d.A) + (long long)b * d.sA;
  const bf16_t* B = d.Btab ? static_cast<const bf16_t*>(d.Btab[b]) : static_cast<const bf16_t*>(d.B) + (long long)b * d.sB;

  f32x16_t acc[TM][TM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  uint4 ra[BT / 32], rb[BT / 32];
  const int KT = (d.K + BK - 1) / BK;

  load_tile_global<BT, A_KS>(ra, A, d.lda, m0, 0, d.M, d.K, tid);
  load_tile_global<BT, B_KS>(rb, B, d.ldb, n0, 0, d.N, d.K, tid);
  store_tile_lds<BT, A_KS>(ra, lds, tid);
  store_tile_lds<BT, B_KS>(rb, lds + A_BYTES, tid);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const char* sa = lds + (kt & 1) * STAGE;
    const char* sb = sa + A_BYTES;
    const bool more = kt + 1 < KT;
    if (more) {
      load_tile_global<BT, A_KS>(ra, A, d.lda, m0, (kt + 1) * BK, d.M, d.K, tid);
      load_tile_global<BT, B_KS>(rb, B, d.ldb, n0, (kt + 1) * BK, d.N, d.K, tid);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8_t af[TM], bfr[TM];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = read_frag<BT, A_KS>(sa, wm * (BT / 2) + i * 32, ks, lane);
#pragma unroll
      for (int j = 0; j < TM; ++j) bfr[j] = read_frag<BT, B_KS>(sb, wn * (BT / 2) + j * 32, ks, lane);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
    }
    if (more) {
      char* na = lds + ((kt + 1) & 1) * STAGE;
      store_tile_lds<BT, A_KS>(ra, na, tid);
      store_tile_lds<BT, B_KS>(rb, na + A_BYTES, tid);
    }
    __syncthreads();
  }

  // ---- epilogue -------------------------------------------------------------------
  // The accumulators go through LDS (the stage buffers are free now), one 32-row band of
  // the wavefront's sub-tile at a time, so that C and E move as 16-byte row segments and
  // the code stays small enough to keep every accumulator index a compile-time constant.
  constexpr int W = BT / 2;          // columns of a wavefront's sub-tile
  constexpr int PITCH = W + 4;       // floats; 16-byte aligned rows, conflict-free float4 writes
  constexpr int CPR = W / 8;         // 8-column chunks per row
  constexpr int RPP = 64 / CPR;      // rows per pass of the wavefront
  float* stg = reinterpret_cast<float*>(lds) + wave * (32 * PITCH);
  const Epi ep{d.s0, d.s1, d.epilogue, d.faithful, d.c_dtype == DA_F32};
  const bool mirror = SYM && (ti != tj);
  const bool has_e = d.epilogue == DA_EPI_AXPBY;
  const int wm0 = m0 + wm * W, wn0 = n0 + wn * W;
  // C and E base pointers of this matrix, as byte addresses (element size depends on c_dtype)
  const int csz = ep.c_f32 ? 4 : 2;
  char* const Cbase = d.Ctab ? static_cast<char*>(d.Ctab[b]) : static_cast<char*>(d.C) + (long long)b * d.sC * csz;
  const char* const Ebase = !has_e ? nullptr
                            : d.Etab ? static_cast<const char*>(d.Etab[b])
                                     : static_cast<const char*>(d.E) + (long long)b * d.sE * csz;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    {
      float* row = stg + (lane & 31) * PITCH + (lane >> 5) * 4;
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq)
          *reinterpret_cast<float4*>(row + j * 32 + vq * 8) =
              make_float4(acc[i][j][vq * 4], acc[i][j][vq * 4 + 1], acc[i][j][vq * 4 + 2], acc[i][j][vq * 4 + 3]);
    }
    __syncthreads();
    const int band_m = wm0 + i * 32;
    for (int pass = 0; pass < 32 / RPP; ++pass) {
      const int r = pass * RPP + lane / CPR;
      const int c8 = (lane % CPR) * 8;
      const int m = band_m + r, n = wn0 + c8;
      if (m < d.M && n < d.N) {
        float* sp = stg + r * PITCH + c8;
        const float4 a0 = *reinterpret_cast<const float4*>(sp);
        const float4 a1 = *reinterpret_cast<const float4*>(sp + 4);
        float v[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        float e[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const long long off = (long long)m * d.ldc + n;
        if (ep.c_f32) {
          if (has_e) {
            const float* Ep = reinterpret_cast<const float*>(Ebase) + (long long)m * d.lde + n;
            const float4 e0 = *reinterpret_cast<const float4*>(Ep);
            const float4 e1 = *reinterpret_cast<const float4*>(Ep + 4);
            e[0] = e0.x; e[1] = e0.y; e[2] = e0.z; e[3] = e0.w; e[4] = e1.x; e[5] = e1.y; e[6] = e1.z; e[7] = e1.w;
          }
#pragma unroll
          for (int q = 0; q < 8; ++q) v[q] = epi_value(ep, v[q], e[q]);
          float* Cp = reinterpret_cast<float*>(Cbase) + off;
          *reinterpret_cast<float4*>(Cp) = make_float4(v[0], v[1], v[2], v[3]);
          *reinterpret_cast<float4*>(Cp + 4) = make_float4(v[4], v[5], v[6], v[7]);
        } else {
          if (has_e) {
            const uint4 ev = *reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(Ebase) + (long long)m * d.lde + n);
            const uint32_t w[4] = {ev.x, ev.y, ev.z, ev.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              e[2 * q] = bf2f((bf16_t)(w[q] & 0xffffu));
              e[2 * q + 1] = bf2f((bf16_t)(w[q] >> 16));
            }
          }
          uint32_t pk[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const bf16_t lo = f2bf(epi_value(ep, v[2 * q], e[2 * q]));
            const bf16_t hi = f2bf(epi_value(ep, v[2 * q + 1], e[2 * q + 1]));
            pk[q] = (uint32_t)lo | ((uint32_t)hi << 16);
            v[2 * q] = bf2f(lo);
            v[2 * q + 1] = bf2f(hi);
          }
          *reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(Cbase) + off) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        }
        if (mirror) {  // keep the final values for the transposed store
          *reinterpret_cast<float4*>(sp) = make_float4(v[0], v[1], v[2], v[3]);
          *reinterpret_cast<float4*>(sp + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
      }
    }
    if (mirror) {
      __syncthreads();
      // C^T: row n of the mirrored tile holds 32 consecutive m of this band
      for (int pass = 0; pass < (W / 64) * 4; ++pass) {
        const int nl = (pass >> 2) * 64 + lane;
        const int mg = (pass & 3) * 8;
        const int n = wn0 + nl, m = band_m + mg;
        if (n < d.N && m < d.M) {  // M is a multiple of 8 for symmetric outputs
          float v[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) v[q] = stg[(mg + q) * PITCH + nl];
          const long long off = (long long)n * d.ldc + m;
          if (ep.c_f32) {
            float* Cp = reinterpret_cast<float*>(Cbase) + off;
            *reinterpret_cast<float4*>(Cp) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4*>(Cp + 4) = make_float4(v[4], v[5], v[6], v[7]);
          } else {
            uint32_t pk[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) pk[q] = (uint32_t)f2bf(v[2 * q]) | ((uint32_t)f2bf(v[2 * q + 1]) << 16);
            *reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(Cbase) + off) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
          }
        }
      }
    }
    __syncthreads();
  }
}

template <int BT, bool A_KS, bool B_KS, bool SYM>
int launch(const GemmDesc& d, hipStream_t stream) {
  constexpr int smem = 2 * (Tile<BT, A_KS>::bytes + Tile<BT, B_KS>::bytes);
  auto kern = gemm_bf16_kernel<BT, A_KS, B_KS, SYM>;
  static bool configured = false;  // benign race: the attribute call is idempotent
  if (!configured) {
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    configured = true;
  }
  const int tiles_m = (d.M + BT - 1) / BT, tiles_n = (d.N + BT - 1) / BT;
  const long long per_batch = SYM ? (long long)tiles_m * (tiles_m + 1) / 2 : (long long)tiles_m * tiles_n;
  const long long blocks = per_batch * d.batch;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return DA_ERR_LIMIT;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), smem, stream, d);
  return da_launch_status();
}

template <int BT>
int dispatch_layout(const GemmDesc& d, hipStream_t stream) {
  if (d.symmetric) return launch<BT, false, false, true>(d, stream);
  if (!d.a_kstrided && !d.b_kstrided) return launch<BT, false, false, false>(d, stream);
  if (!d.a_kstrided && d.b_kstrided) return launch<BT, false, true, false>(d, stream);
  if (d.a_kstrided && !d.b_kstrided) return launch<BT, true, false, false>(d, stream);
  return launch<BT, true, true, false>(d, stream);
}

}  // namespace

// Alignment contract: K, N, every leading dimension and every batch stride are multiples
// of 8 elements (16-byte chunks); M too when A is k-strided; pointers 16-byte aligned.
int da_gemm_bf16(const GemmDesc& d, hipStream_t stream) {
  if ((!d.A && !d.Atab) || (!d.B && !d.Btab) || (!d.C && !d.Ctab) || d.M <= 0 || d.N <= 0 || d.K <= 0 || d.batch <= 0) return DA_ERR_ARG;
  if (d.epilogue == DA_EPI_AXPBY && !d.E && !d.Etab) return DA_ERR_ARG;
  if (d.c_dtype != DA_BF16 && d.c_dtype != DA_F32) return DA_ERR_DTYPE;
  if ((d.K | d.N | d.lda | d.ldb | d.ldc) & 7) return DA_ERR_ALIGN;
  if ((d.sA | d.sB | d.sC) & 7) return DA_ERR_ALIGN;
  if ((d.E || d.Etab) && ((d.lde & 7) || (d.sE & 7))) return DA_ERR_ALIGN;
  if (d.a_kstrided && (d.M & 7)) return DA_ERR_ALIGN;
  if (((uintptr_t)d.A | (uintptr_t)d.B | (uintptr_t)d.C | (uintptr_t)d.E) & 15) return DA_ERR_ALIGN;
  if (d.symmetric && (d.M != d.N || d.a_kstrided || d.b_kstrided)) return DA_ERR_ARG;
  // Large tiles once there are enough of them to cover the 256 CUs; small tiles otherwise.
  const long long t256 = (long long)((d.M + 255) / 256) * ((d.N + 255) / 256) * d.batch / (d.symmetric ? 2 : 1);
  if (d.M >= 1024 && d.N >= 1024 && t256 >= 200) return dispatch_layout<256>(d, stream);
  return dispatch_layout<128>(d, stream);
}
