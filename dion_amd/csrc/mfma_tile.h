// Device-side building blocks shared by the bf16 matrix-core kernels: LDS tile layouts and their swizzles,
// MFMA fragment reads, direct-to-LDS loads, and the rounding-faithful epilogue arithmetic.
#pragma once
#include "common.h"

namespace {

typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

constexpr int BK = 64;       // k elements per stage

// Physical 16-byte chunk of a k-contiguous tile row ([BT][8 chunks]) and of a k-strided tile
// row ([64][BT/8 chunks], 32-byte slots swizzled with the k-row).
__device__ __forceinline__ int kc_swizzle(int chunk, int row) { return chunk ^ ((row >> 1) & 7); }
__device__ __forceinline__ int ks_swizzle(int chunk, int krow) { return (((chunk >> 1) ^ (krow & 3)) << 1) | (chunk & 1); }

// Fragment of 32 rows x 16 k for one MFMA: lane l gets row (l & 31), k = 8 * (l >> 5) .. +8.
template <int BT, bool KS>
__device__ __forceinline__ bf16x8_t read_frag(const char* lds, int r0, int ks, int lane) {
  if (!KS) {
    const int row = r0 + (lane & 31);
    const int phys = kc_swizzle(ks * 2 + (lane >> 5), row);
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(lds + row * 128 + phys * 16);
    return __builtin_bit_cast(bf16x8_t, v);
  } else {
    // Per 16-lane group g: rows r0 + 16 * (g & 1) .. +16, k-group g >> 1.  The four lanes
    // 4q .. 4q+3 of a group together supply 16 consecutive rows of k-row q; the transpose
    // read returns to lane i of the group the four k values of row i.  The 32-byte slot a
    // group reads is swizzled with (k-row & 3) = q, so its four k-rows hit different banks.
    const int g = lane >> 4;
    const int q = (lane & 15) >> 2;
    const int slot = ((r0 >> 4) + (g & 1)) ^ q;
    const int kr = ks * 16 + (g >> 1) * 8 + q;
    const char* p = lds + kr * (BT * 2) + slot * 32 + (lane & 3) * 8;
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(DA_LDS_PTR(s16x4_t, p));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(DA_LDS_PTR(s16x4_t, p + 4 * (BT * 2)));
    typedef short s16x8_t __attribute__((ext_vector_type(8)));
    const s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, v);
  }
}

// Fragment of 16 rows x 32 k for one v_mfma_f32_16x16x32_bf16: lane l gets row (l & 15), k = 8 * (l >> 4) .. +8 of
// the 32-deep k-step `ks` (0 or 1) of a stage.
template <int BT, bool KS>
__device__ __forceinline__ bf16x8_t read_frag16(const char* lds, int r0, int ks, int lane) {
  if (!KS) {
    const int row = r0 + (lane & 15);
    const int phys = kc_swizzle(ks * 4 + (lane >> 4), row);
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(lds + row * 128 + phys * 16);
    return __builtin_bit_cast(bf16x8_t, v);
  } else {
    // All four 16-lane groups read the same 16 rows, group g the k-rows 8 g .. 8 g + 7: the four lanes 4q .. 4q+3
    // supply the 16 rows of k-row q (then q + 4), and the transpose read hands lane i the four k values of row i.
    const int g = lane >> 4;
    const int q = (lane & 15) >> 2;
    const int slot = (r0 >> 4) ^ q;
    const int kr = ks * 32 + g * 8 + q;
    const char* p = lds + kr * (BT * 2) + slot * 32 + (lane & 3) * 8;
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(DA_LDS_PTR(s16x4_t, p));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(DA_LDS_PTR(s16x4_t, p + 4 * (BT * 2)));
    typedef short s16x8_t __attribute__((ext_vector_type(8)));
    const s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, v);
  }
}

__device__ __forceinline__ int wave_uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// 16 bytes per lane from global memory straight into LDS: lane p's data lands at LDS byte
// address `l + 16 p`.  `base` and `l` are wave-uniform, `off` is the lane's byte offset.
// Written as assembly on purpose: with the compiler's own LDS-DMA intrinsic in the loop, its
// wait-count insertion degrades every LDS-read wait to lgkmcnt(0), which serialises the
// fragment reads of k-step s+1 with the MFMAs of k-step s.  The price is that the compiler
// does not know about these loads: dma_wait() must precede the barrier that publishes a stage.
// The s_nop covers the M0-write -> LDS-DMA and the VALU-SGPR-write -> VMEM-address hazards,
// which the hazard recogniser cannot see inside an asm block.
// (M0 is not in the clobber list -- the compiler rejects reserved registers there; nothing else
// in this kernel keeps a value in M0.)
__device__ __forceinline__ void dma16(const char* base, unsigned off, unsigned l) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(base);
  const unsigned long long u = ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(a >> 32)) << 32) |
                               (unsigned)__builtin_amdgcn_readfirstlane((int)a);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 4\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(off), "s"(u), "s"(__builtin_amdgcn_readfirstlane((int)l))
               : "memory");
}
__device__ __forceinline__ void dma_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ unsigned lds_addr(const char* p) {
  return (unsigned)(uintptr_t)DA_LDS_PTR(const char, p);
}

// value of C from the accumulator and (optionally) the epilogue operand; the final rounding to
// C's dtype happens at the store
template <bool HAS_E, bool FAITHFUL, bool CF32>
__device__ __forceinline__ float epi_value(float s0, float s1, float acc, float e) {
  if (FAITHFUL) {
    float t = rbf(acc);
    t = rbf(s1 * t);
    if (HAS_E) {
      float u = s0 * e;
      if (!CF32) u = rbf(u);
      t = u + t;
    }
    return t;
  }
  return HAS_E ? s0 * e + s1 * acc : s1 * acc;
}

// Two neighbouring elements of a bf16 C at once.  Written with explicit pairs because the epilogue is bound by
// its VALU instructions (a 256 x 256 tile has 128 elements per lane): converting element by element the
// compiler issues one v_cvt_pk_bf16_f32 per value and 25 instructions per pair for the rounding-faithful
// a X + B X form; with both halves of every conversion used, and the exact multiplication by s1 == 1 skipped,
// it is 13 (and a single conversion for a plain rounded store).  S1_ONE: s1 == 1 (a compile-time variant).
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned cvt_pk_bf16(float a, float b) {
  const f32x2_t f = {a, b};
  const bf16x2_t h = __builtin_convertvector(f, bf16x2_t);
  return __builtin_bit_cast(unsigned, h);
}
__device__ __forceinline__ float lo_f(unsigned w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float hi_f(unsigned w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// The value pair of epi_value<HAS_E, FAITHFUL, false>, rounded to bf16 and packed (`ew`: the two bf16 of E).
template <bool HAS_E, bool FAITHFUL, bool S1_ONE>
__device__ __forceinline__ unsigned epi_pair(float s0, float s1, float a0, float a1, unsigned ew) {
  if (FAITHFUL) {
    unsigned p = cvt_pk_bf16(a0, a1);
    if (!S1_ONE) p = cvt_pk_bf16(s1 * lo_f(p), s1 * hi_f(p));
    if (!HAS_E) return p;
    const unsigned q = cvt_pk_bf16(s0 * lo_f(ew), s0 * hi_f(ew));
    return cvt_pk_bf16(lo_f(q) + lo_f(p), hi_f(q) + hi_f(p));
  }
  if (HAS_E) return cvt_pk_bf16(s0 * lo_f(ew) + s1 * a0, s0 * hi_f(ew) + s1 * a1);
  return cvt_pk_bf16(s1 * a0, s1 * a1);
}

typedef __attribute__((address_space(1))) u32x4_t global_u32x4_t;
__device__ __forceinline__ u32x4_t ldg16(const char* p) { return *(const global_u32x4_t*)p; }
__device__ __forceinline__ void stg16(char* p, u32x4_t v) { *(global_u32x4_t*)p = v; }

__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

}  // namespace
