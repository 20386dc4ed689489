// One output tile of the bf16 matrix-core GEMM as device code shared by the kernels that run it: the batched /
// grouped GEMM kernel (one workgroup per tile, gemm_bf16.hip) and the persistent Newton-Schulz kernel (a workgroup
// takes tile after tile of the products of a whole iteration sequence, ns_flow.hip).
//
// Work decomposition, LDS layouts, direct-to-LDS staging, operand-swapped MFMA and the epilogue through LDS are
// described at the top of gemm_bf16.hip.
#pragma once
#include "common.h"
#include "mfma_tile.h"

namespace {

// MI: edge of the MFMA's output block -- 32: v_mfma_f32_32x32x16_bf16 (16 accumulator registers per block, 16-deep
// k-steps), 16: v_mfma_f32_16x16x32_bf16 (4 registers, 32-deep k-steps; the chip holds a higher clock under it).
template <int MI> struct AccOf;
template <> struct AccOf<32> { typedef f32x16_t type; };
template <> struct AccOf<16> { typedef f32x4_t type; };

#ifndef DA_MI
#define DA_MI 16   // the MFMA shape the kernels of this library are built with (32: the 32x32x16 form)
#endif
#ifndef DA_KLOOP_ABLATE
#define DA_KLOOP_ABLATE 0   // see gemm_tile_k_loop: measurement builds only
#endif

template <int BT_, int WGM_, int WGN_, int MI_ = DA_MI>
struct Cfg {
  static constexpr int BT = BT_, WGM = WGM_, WGN = WGN_, MI = MI_;
  static constexpr int NT = 64 * WGM * WGN;        // threads
  static constexpr int TMI = BT / (MI * WGM);      // accumulator blocks per wavefront, row direction
  static constexpr int TNJ = BT / (MI * WGN);      // ... column direction
  static constexpr int AV = MI * MI / 64;          // accumulator registers per block
  static constexpr int NCH = BT * 8 / NT;          // 16-byte chunks per thread per operand stage
  static constexpr int WROWS = BT / WGM, WCOLS = BT / WGN;
  static constexpr int NB = WROWS / 32;            // 32-row bands of a wavefront's sub-tile (the epilogue's unit)
  typedef typename AccOf<MI>::type acc_t;
};

template <int BT, bool KS>
struct Tile {
  static constexpr int bytes = BT * BK * 2;   // either layout: 64 x BT bf16
};

// Per-thread addressing of the NCH 16-byte chunks a thread moves per operand stage.
//   Register-staged path (bounds-checked): chunk i lies at global `g + i * gstep` (elements)
//   and goes to LDS byte offset `l + i * lstep`.
//   Direct-to-LDS path: wave-instruction i of wavefront w fills the 1024-byte LDS block
//   (i * NW + w); lane p of it fetches the chunk whose *physical* position is p, i.e. the
//   swizzle is applied to the global address, which is kept as a wave-uniform base pointer
//   (`dbase`) plus a 32-bit byte offset (`doff + i * dstep`, per lane and loop invariant, plus
//   the stage's offset, a scalar) so that the loads use SGPR-base addressing.
template <typename C, bool KS>
struct StageAddr {
  const bf16_t* g;
  const char* dbase;
  unsigned doff, dstep;
  long long gstep, tstep;   // per chunk and per stage, in elements
  int l, lstep;
  int row, col;             // first chunk's (row within tile, k offset) resp. (k row, row offset)
  // `dim`: extent of the operand in the tile's row direction (M or N); the direct-to-LDS addresses of a
  // k-strided operand keep their 16-byte chunks inside it (an edge tile then fetches a neighbouring chunk for the
  // columns it does not own: finite values that the bounds-checked epilogue never stores).
  __device__ __forceinline__ StageAddr(const bf16_t* base, int ld, int row0, int tid, int dim) {
    constexpr int NW = C::NT / 64;
    const int lane = tid & 63, wave = tid >> 6;
    if (!KS) {
      row = tid >> 3;
      col = (tid & 7) * 8;
      g = base + (long long)(row0 + row) * ld + col;
      gstep = (long long)(C::NT / 8) * ld;
      tstep = BK;
      l = row * 128 + kc_swizzle(tid & 7, row) * 16;
      lstep = (C::NT / 8) * 128;   // NT/8 is a multiple of 16: the swizzle term is the same for all chunks
      const int drow = wave * 8 + (lane >> 3);             // block (0 * NW + wave), 8 rows per block
      dbase = reinterpret_cast<const char*>(base + (long long)row0 * ld);
      doff = (unsigned)(drow * ld + kc_swizzle(lane & 7, drow) * 8) * 2u;
      dstep = (unsigned)(NW * 8 * ld) * 2u;                // NW * 8 is a multiple of 16
    } else {
      constexpr int CPR = C::BT / 8;                       // chunks per k-row
      constexpr int RPB = 64 / CPR;                        // k-rows per 1024-byte block
      row = tid / CPR;
      col = (tid % CPR) * 8;
      g = base + (long long)row * ld + row0 + col;
      gstep = (long long)(C::NT / CPR) * ld;
      tstep = (long long)BK * ld;
      l = row * (C::BT * 2) + ks_swizzle(tid % CPR, row) * 16;
      lstep = (C::NT / CPR) * (C::BT * 2);                 // NT / CPR = 16: swizzle term unchanged
      const int drow = wave * RPB + lane / CPR;
      dbase = reinterpret_cast<const char*>(base + row0);
      int dcol = ks_swizzle(lane % CPR, drow) * 8;
      if (row0 + dcol > dim - 8) dcol = dim - 8 - row0;
      doff = (unsigned)(drow * ld + dcol) * 2u;
      dstep = (unsigned)(NW * RPB * ld) * 2u;              // NW * RPB = 16
    }
  }
};

// The accumulators go through LDS (the stage buffers are free by now), one 32-row band of the
// wavefront's sub-tile at a time, so that C and E move as 16-byte row segments.  Each wavefront
// stages through its own LDS region, so only wavefront-level ordering is needed inside.
// Output dtype, epilogue form and rounding mode are compile-time here: evaluated per element at
// run time they cost more than the MFMAs of a short-K product.
// The weight update of the reference's post-orthogonalisation pass on 8 consecutive elements of the weights at `Wp`
// (dion/muon.py:569-573): W <- r_W(r_W(W * decay) - r_bf16(U * step)), U = the eight bf16 results in `pk`; the old
// weights come in x0 (bf16: all eight) resp. x0, x1 (fp32), requested a band earlier.
__device__ __forceinline__ void update_weights8(char* Wp, bool w_f32, u32x4_t x0, u32x4_t x1, u32x4_t pk, float decay,
                                                float step) {
  if (!w_f32) {
    u32x4_t o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned x = x0[q], u = pk[q];
      const unsigned xd = cvt_pk_bf16(lo_f(x) * decay, hi_f(x) * decay);
      const unsigned t = cvt_pk_bf16(lo_f(u) * step, hi_f(u) * step);
      o[q] = cvt_pk_bf16(lo_f(xd) - lo_f(t), hi_f(xd) - hi_f(t));
    }
    stg16(Wp, o);
  } else {
    u32x4_t o0, o1;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned u = pk[q];
      const unsigned t = cvt_pk_bf16(lo_f(u) * step, hi_f(u) * step);
      const unsigned xa = q < 2 ? x0[2 * q] : x1[2 * q - 4], xb = q < 2 ? x0[2 * q + 1] : x1[2 * q - 3];
      const float ra = __builtin_bit_cast(float, xa) * decay - lo_f(t);
      const float rb = __builtin_bit_cast(float, xb) * decay - hi_f(t);
      if (q < 2) { o0[2 * q] = __builtin_bit_cast(unsigned, ra); o0[2 * q + 1] = __builtin_bit_cast(unsigned, rb); }
      else { o1[2 * q - 4] = __builtin_bit_cast(unsigned, ra); o1[2 * q - 3] = __builtin_bit_cast(unsigned, rb); }
    }
    stg16(Wp, o0);
    stg16(Wp + 16, o1);
  }
}

// UPD: 0 the result is stored in C; 1 / 2 it is not stored but updates the weights d.upd_tab[b] in place (2: those are
// stored transposed), see GemmDesc.
template <typename C, bool SYM, bool FULL, bool CF32, bool HAS_E, bool FAITHFUL, bool S1_ONE, int UPD = 0, bool WF32 = false>
__device__ __forceinline__ void epilogue_impl(typename C::acc_t (&acc)[C::TMI][C::TNJ], const GemmDesc& d, char* lds, int b,
                                              bool mirror, int m0, int n0, int wave, int lane, int wm, int wn) {
  constexpr int W = C::WCOLS;        // columns of a wavefront's sub-tile
  constexpr int PITCH = W + 4;       // floats; 16-byte aligned rows, conflict-free float4 writes
  constexpr int CPR = W / 8;         // 8-column chunks per row
  constexpr int RPP = 64 / CPR;      // rows per pass of the wavefront
  constexpr int NPASS = 32 / RPP;
  constexpr int CSZ = CF32 ? 4 : 2;
  constexpr int NV = CF32 ? 2 : 1;   // 16-byte vectors per 8 elements
  float* stg = reinterpret_cast<float*>(lds) + wave * (32 * PITCH);
  // the descriptor lives in the kernel-argument segment: fields read inside the band loop would be fetched
  // again after every store (scalar load + a full wait in the middle of the band), so they are copied first
  const float s0 = d.s0, s1 = d.s1;
  const long long c2 = (!HAS_E && !FAITHFUL && !SYM && !CF32) ? d.c2_off * 2 : 0;   // bytes to the second output
  const int dM = d.M, dN = d.N;
  const long long ldc = d.ldc, lde = d.lde;
  const int wm0 = m0 + wm * C::WROWS, wn0 = n0 + wn * W;
  char* const Cbase = d.Ctab ? static_cast<char*>(d.Ctab[b]) : static_cast<char*>(d.C) + (long long)b * d.sC * CSZ;
  const char* const Ebase = !HAS_E ? nullptr
                            : d.Etab ? static_cast<const char*>(d.Etab[b])
                                     : static_cast<const char*>(d.E) + (long long)b * d.sE * CSZ;
  const int lr = lane / CPR, c8 = (lane % CPR) * 8;
  const bool col_ok = FULL || wn0 + c8 < dN;
  char* const Wbase = UPD ? static_cast<char*>(d.upd_tab[b]) : nullptr;
  constexpr bool w_f32 = WF32;   // (a compile-time variant: the prefetch buffers differ in size)
  constexpr int wsz = w_f32 ? 4 : 2;
  const long long ldw = d.upd_ld;
  const float w_decay = d.upd_decay, w_step = d.upd_step;
  // E is requested up to three bands ahead (registers that the K loop's fragments no longer need), so that a
  // tile's epilogue pays one memory latency and not one per band; an fp32 E (twice the registers) one band ahead.
  constexpr int DEPTH = (!HAS_E || CF32) ? 1 : (UPD ? 2 : (C::NB < 3 ? C::NB : 3));
  u32x4_t ev[DEPTH][NPASS][NV];
  // the weights a band updates are requested when the band starts, ahead of its staging through LDS and of the
  // arithmetic on E (two vectors per 8 elements when they are fp32)
  constexpr int NWP = UPD == 2 ? (W / 64) * 4 : NPASS;
  constexpr int NWV = WF32 ? 2 : 1;
  u32x4_t wv[NWP][NWV];
  auto weight_ptr = [&](int band, int pass) -> char* {
    if (UPD == 2) {
      const int n = wn0 + (pass >> 2) * 64 + lane, m = wm0 + band * 32 + (pass & 3) * 8;
      return Wbase + ((long long)n * ldw + m) * wsz;
    }
    const int m = wm0 + band * 32 + pass * RPP + lr;
    return Wbase + ((long long)m * ldw + wn0 + c8) * wsz;
  };
  auto load_w = [&](int band, u32x4_t (&dst)[NWP][NWV]) {
#pragma unroll
    for (int pass = 0; pass < NWP; ++pass) {
      const char* p = weight_ptr(band, pass);
#pragma unroll
      for (int h = 0; h < NWV; ++h) dst[pass][h] = ldg16(p + 16 * h);
    }
  };

  auto load_e = [&](int band, u32x4_t (&dst)[NPASS][NV]) {
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
      const int m = wm0 + band * 32 + pass * RPP + lr;
      const u32x4_t z = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int h = 0; h < NV; ++h) dst[pass][h] = z;
      if (col_ok && (FULL || m < dM)) {
        const char* Ep = Ebase + ((long long)m * lde + wn0 + c8) * CSZ;
#pragma unroll
        for (int h = 0; h < NV; ++h) dst[pass][h] = ldg16(Ep + 16 * h);
      }
    }
  };
  if (HAS_E) {
#pragma unroll
    for (int q = 0; q < DEPTH; ++q) load_e(q, ev[q]);
  }
#pragma unroll
  for (int i = 0; i < C::NB; ++i) {
    if (UPD) load_w(i, wv);
    if (C::MI == 32) {
      float* row = stg + (lane & 31) * PITCH + (lane >> 5) * 4;
#pragma unroll
      for (int j = 0; j < C::TNJ; ++j)
#pragma unroll
        for (int vq = 0; vq < C::AV / 4; ++vq)
          *reinterpret_cast<float4*>(row + j * 32 + vq * 8) =
              make_float4(acc[i][j][vq * 4], acc[i][j][vq * 4 + 1], acc[i][j][vq * 4 + 2], acc[i][j][vq * 4 + 3]);
    } else {
      // 16 x 16 blocks: a lane holds, for row (lane & 15) of a block, the four columns 4 (lane >> 4) .. + 3
      float* row = stg + (lane & 15) * PITCH + (lane >> 4) * 4;
#pragma unroll
      for (int ib = 0; ib < 2; ++ib)
#pragma unroll
        for (int j = 0; j < C::TNJ; ++j) {
          const typename C::acc_t& a = acc[(2 * i + ib) % C::TMI][j];
          *reinterpret_cast<float4*>(row + ib * 16 * PITCH + j * 16) = make_float4(a[0], a[1], a[2], a[3]);
        }
    }
    wave_sync_lds();
    const int band_m = wm0 + i * 32;
    u32x4_t ec[NPASS][NV];
    if (HAS_E) {
#pragma unroll
      for (int pass = 0; pass < NPASS; ++pass)
#pragma unroll
        for (int h = 0; h < NV; ++h) ec[pass][h] = ev[i % DEPTH][pass][h];
      if (i + DEPTH < C::NB) load_e(i + DEPTH, ev[i % DEPTH]);
    }

#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
      const int r = pass * RPP + lr;
      const int m = band_m + r;
      if (col_ok && (FULL || m < dM)) {
        float* sp = stg + r * PITCH + c8;
        const float4 a0 = *reinterpret_cast<const float4*>(sp);
        const float4 a1 = *reinterpret_cast<const float4*>(sp + 4);
        float v[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        float e[8];
        char* Cp = Cbase + ((long long)m * ldc + wn0 + c8) * CSZ;
        if (CF32) {
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const unsigned w = HAS_E ? ec[pass][q >> 2][q & 3] : 0u;  // (bit_cast of a vector element lvalue reads element 0)
            e[q] = __builtin_bit_cast(float, w);
          }
#pragma unroll
          for (int q = 0; q < 8; ++q) v[q] = epi_value<HAS_E, FAITHFUL, true>(s0, s1, v[q], e[q]);
          const u32x4_t o0 = {__builtin_bit_cast(unsigned, v[0]), __builtin_bit_cast(unsigned, v[1]),
                              __builtin_bit_cast(unsigned, v[2]), __builtin_bit_cast(unsigned, v[3])};
          const u32x4_t o1 = {__builtin_bit_cast(unsigned, v[4]), __builtin_bit_cast(unsigned, v[5]),
                              __builtin_bit_cast(unsigned, v[6]), __builtin_bit_cast(unsigned, v[7])};
          stg16(Cp, o0);
          stg16(Cp + 16, o1);
        } else {
          u32x4_t pk;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const unsigned w = HAS_E ? ec[pass][0][q] : 0u;   // (copied out: see the note on bit_cast above)
            const unsigned o = epi_pair<HAS_E, FAITHFUL, S1_ONE>(s0, s1, v[2 * q], v[2 * q + 1], w);
            pk[q] = o;
            if (SYM) {
              v[2 * q] = lo_f(o);
              v[2 * q + 1] = hi_f(o);
            }
          }
          if (UPD == 0) stg16(Cp, pk);
          if (UPD == 1) update_weights8(weight_ptr(i, pass), w_f32, wv[pass][0], wv[pass][NWV - 1], pk, w_decay, w_step);
          if (UPD == 2) {   // the final values stay in the staging area for the transposed pass below
            *reinterpret_cast<float4*>(sp) = make_float4(lo_f(pk[0]), hi_f(pk[0]), lo_f(pk[1]), hi_f(pk[1]));
            *reinterpret_cast<float4*>(sp + 4) = make_float4(lo_f(pk[2]), hi_f(pk[2]), lo_f(pk[3]), hi_f(pk[3]));
          }
          if (!HAS_E && !FAITHFUL && !SYM && c2) {
            // what the stored bf16 leaves of s1 * acc, as a second bf16 matrix
            u32x4_t lo;
#pragma unroll
            for (int q = 0; q < 4; ++q) lo[q] = cvt_pk_bf16(s1 * v[2 * q] - lo_f(pk[q]), s1 * v[2 * q + 1] - hi_f(pk[q]));
            stg16(Cp + c2, lo);
          }
        }
        if (SYM && mirror) {  // keep the final values for the transposed store
          *reinterpret_cast<float4*>(sp) = make_float4(v[0], v[1], v[2], v[3]);
          *reinterpret_cast<float4*>(sp + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
      }
    }
    if (UPD == 2) {
      wave_sync_lds();
      // the weights are stored transposed: row n of W holds 32 consecutive m of this band
#pragma unroll
      for (int pass = 0; pass < (W / 64) * 4; ++pass) {
        const int nl = (pass >> 2) * 64 + lane;
        const int mg = (pass & 3) * 8;
        const int n = wn0 + nl, m = band_m + mg;
        if (FULL || (n < dN && m < dM)) {
          u32x4_t pk;
#pragma unroll
          for (int q = 0; q < 4; ++q) pk[q] = cvt_pk_bf16(stg[(mg + 2 * q) * PITCH + nl], stg[(mg + 2 * q + 1) * PITCH + nl]);
          update_weights8(weight_ptr(i, pass), w_f32, wv[pass][0], wv[pass][NWV - 1], pk, w_decay, w_step);
        }
      }
    }
    if (SYM && mirror) {
      wave_sync_lds();
      // C^T: row n of the mirrored tile holds 32 consecutive m of this band
#pragma unroll
      for (int pass = 0; pass < (W / 64) * 4; ++pass) {
        const int nl = (pass >> 2) * 64 + lane;
        const int mg = (pass & 3) * 8;
        const int n = wn0 + nl, m = band_m + mg;
        if (FULL || (n < dN && m < dM)) {  // M is a multiple of 8 for symmetric outputs
          float v[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) v[q] = stg[(mg + q) * PITCH + nl];
          char* Cp = Cbase + ((long long)n * ldc + m) * CSZ;
          if (CF32) {
            const u32x4_t o0 = {__builtin_bit_cast(unsigned, v[0]), __builtin_bit_cast(unsigned, v[1]),
                                __builtin_bit_cast(unsigned, v[2]), __builtin_bit_cast(unsigned, v[3])};
            const u32x4_t o1 = {__builtin_bit_cast(unsigned, v[4]), __builtin_bit_cast(unsigned, v[5]),
                                __builtin_bit_cast(unsigned, v[6]), __builtin_bit_cast(unsigned, v[7])};
            stg16(Cp, o0);
            stg16(Cp + 16, o1);
          } else {
            u32x4_t pk;
#pragma unroll
            for (int q = 0; q < 4; ++q) pk[q] = cvt_pk_bf16(v[2 * q], v[2 * q + 1]);
            stg16(Cp, pk);
          }
        }
      }
    }
    wave_sync_lds();
  }
}

template <typename C, bool SYM, bool FULL>
__device__ __forceinline__ void epilogue(typename C::acc_t (&acc)[C::TMI][C::TNJ], const GemmDesc& d, char* lds, int b, int ti,
                                         int tj, int m0, int n0, int wave, int lane, int wm, int wn) {
  const bool mirror = SYM && (ti != tj);
  const bool cf32 = d.c_dtype == DA_F32, has_e = d.epilogue == DA_EPI_AXPBY, fa = d.faithful != 0;
  const bool one = d.s1 == 1.f;   // rounding-faithful bf16 output: the exact multiplication by 1 is left out
#define DA_EPI(CF, HE, FA, S1) \
  epilogue_impl<C, SYM, FULL, CF, HE, FA, S1>(acc, d, lds, b, mirror, m0, n0, wave, lane, wm, wn)
#define DA_EPI_UPD(FA, S1, U, WF) \
  epilogue_impl<C, false, FULL, false, true, FA, S1, U, WF>(acc, d, lds, b, false, m0, n0, wave, lane, wm, wn)
#define DA_EPI_UPD_FA(U, WF)                                                              \
  do {                                                                                    \
    if (fa) { if (one) DA_EPI_UPD(true, true, U, WF); else DA_EPI_UPD(true, false, U, WF); } \
    else DA_EPI_UPD(false, false, U, WF);                                                 \
  } while (0)
  if (!SYM && FULL && !cf32 && has_e && d.upd_tab) {
    // (the launcher only sets upd_tab where these conditions hold)
    const bool wf = d.upd_dtype == DA_F32;
    if (d.upd_transposed) { if (wf) DA_EPI_UPD_FA(2, true); else DA_EPI_UPD_FA(2, false); }
    else                  { if (wf) DA_EPI_UPD_FA(1, true); else DA_EPI_UPD_FA(1, false); }
    return;
  }
  if (!cf32) {
    if (has_e) {
      if (fa) { if (one) DA_EPI(false, true, true, true); else DA_EPI(false, true, true, false); }
      else DA_EPI(false, true, false, false);
    } else {
      if (fa) { if (one) DA_EPI(false, false, true, true); else DA_EPI(false, false, true, false); }
      else DA_EPI(false, false, false, false);
    }
  } else {
    if (has_e) { if (fa) DA_EPI(true, true, true, false); else DA_EPI(true, true, false, false); }
    else       { if (fa) DA_EPI(true, false, true, false); else DA_EPI(true, false, false, false); }
  }
#undef DA_EPI
#undef DA_EPI_UPD
#undef DA_EPI_UPD_FA
}


constexpr int DA_LOOP_CHECKED = 0, DA_LOOP_INTERIOR = 1, DA_LOOP_EDGE = 2;

// K loop of one BT x BT tile: acc += sum over dK elements of k of A-rows (m0 ...) x B-rows (n0 ...).  `A`, `B`: the
// matrix's operands at the first k of the sum.  Three forms (MODE):
//   DA_LOOP_INTERIOR: every tile is interior (M, N multiples of BT, K a multiple of 64).  Stages are
//     fetched with direct-to-LDS loads issued one stage ahead; the only wait is the
//     vmcnt(0) in front of the per-stage barrier.  No bounds checks anywhere.
//   DA_LOOP_EDGE: the same K loop for products whose ragged dimension belongs to a k-strided operand (its chunks
//     are kept inside the matrix) and whose other operand has whole tiles; the epilogue checks bounds.  Dion's
//     rank-r products at a rank that is not a multiple of the tile edge (r = 192).
//   DA_LOOP_CHECKED: bounds-checked 16-byte loads into registers (out-of-range chunks zero filled),
//     written to LDS after the stage's MFMAs.
// Ends with a workgroup barrier: the stage buffers are free for the epilogue.
// `after_first_stage` (direct-to-LDS forms) is called once, behind the barrier that publishes the first stage: every
// wavefront has waited for all of its outstanding memory operations by then, stores of earlier work included.
// `same_panel` (direct-to-LDS forms, both operands k-contiguous): the two operands are the same rows of the same
// matrix -- a diagonal tile of X X^T or A A -- so one panel is staged and both fragment sets are read from it.
struct DaNoHook { __device__ __forceinline__ void operator()() const {} };
template <typename C, bool A_KS, bool B_KS, int MODE, typename Hook = DaNoHook>
__device__ __forceinline__ void gemm_tile_k_loop(typename C::acc_t (&acc)[C::TMI][C::TNJ], const GemmDesc& d, const bf16_t* A,
                                                 const bf16_t* B, int dK, int m0, int n0, char* lds, int tid, int lane,
                                                 int wave, int wm, int wn, Hook after_first_stage = Hook(),
                                                 bool same_panel = false) {
  constexpr bool FULL = MODE != DA_LOOP_CHECKED;   // the direct-to-LDS K loop
  constexpr int BT = C::BT, TMI = C::TMI, TNJ = C::TNJ, NCH = C::NCH, NW = C::NT / 64;
  constexpr int A_BYTES = Tile<BT, A_KS>::bytes;
  constexpr int B_BYTES = Tile<BT, B_KS>::bytes;
  constexpr int STAGE = A_BYTES + B_BYTES;
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNJ; ++j)
#pragma unroll
      for (int v = 0; v < C::AV; ++v) acc[i][j][v] = 0.f;

  StageAddr<C, A_KS> sa(A, d.lda, m0, tid, d.M);
  StageAddr<C, B_KS> sb(B, d.ldb, n0, tid, d.N);
  const int ar0 = wm * C::WROWS, br0 = wn * C::WCOLS;
  const int KT = (dK + BK - 1) / BK;
  bf16x8_t fa[C::MI == 32 ? TMI : 1], fb[C::MI == 32 ? TNJ : 1];   // (the 16 x 16 form keeps its own sets below)

  const int b_at = (FULL && !A_KS && !B_KS && same_panel) ? 0 : A_BYTES;   // where the column operand's panel lies in a stage
  if constexpr (C::MI == 32) {
#define DA_FREAD(st, ks)                                                                           \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        fa[i] = read_frag<BT, A_KS>((st), ar0 + i * 32, (ks), lane);                               \
    _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                                \
        fb[j] = read_frag<BT, B_KS>((st) + b_at, br0 + j * 32, (ks), lane);                        \
  } while (0)
#define DA_FREAD2(st, ks, FA, FB)                                                                  \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        FA[i] = read_frag<BT, A_KS>((st), ar0 + i * 32, (ks), lane);                               \
    _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                                \
        FB[j] = read_frag<BT, B_KS>((st) + b_at, br0 + j * 32, (ks), lane);                        \
  } while (0)
#define DA_MMA2(FA, FB)                                                                            \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                            \
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FB[j], FA[i], acc[i][j], 0, 0, 0); \
  } while (0)
#define DA_MMA()                                                                                   \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                            \
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0); \
  } while (0)

  if (FULL) {
// one stage of both operands, straight into LDS: NCH wave-instructions of 1024 bytes each
#define DA_DMA(st)                                                                                 \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        dma16(sa.dbase, sa.doff + i * sa.dstep + koff_a, lds_addr(st) + (i * NW + wave) * 1024);   \
    if (b_at != 0) {                                                                               \
      _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                              \
          dma16(sb.dbase, sb.doff + i * sb.dstep + koff_b, lds_addr(st) + A_BYTES + (i * NW + wave) * 1024); \
    }                                                                                              \
    koff_a += (unsigned)(sa.tstep * 2);                                                            \
    if (koff_a == wrap_a) koff_a = 0;                                                              \
    koff_b += (unsigned)(sb.tstep * 2);                                                            \
  } while (0)
    unsigned koff_a = 0, koff_b = 0;   // byte offset of the stage within the operand (< 4 GiB: checked by the launcher)
    const unsigned wrap_a = (unsigned)d.a_kwrap * 2u;   // A read again from its first column (0: never, koff_a > 0 here)
    DA_DMA(lds);
    dma_wait();
    __syncthreads();
    after_first_stage();
    // Fragments are double buffered in registers: the ds_reads of k-step s+1 are issued before
    // the MFMAs of k-step s (scheduling fences keep the compiler from sinking them back down to
    // their first use), and the stage barrier sits before the last k-step so that the first
    // fragments of the next stage are fetched under the last MFMAs of this one.
    bf16x8_t ga[TMI], gb[TNJ];
    DA_FREAD(lds, 0);
    for (int kt = 0; kt < KT; ++kt) {
      char* cur = lds + (kt & 1) * STAGE;
      char* nxt = lds + ((kt + 1) & 1) * STAGE;
      const bool more = kt + 1 < KT;
      if (more) DA_DMA(nxt);
      DA_FREAD2(cur, 1, ga, gb);
      __builtin_amdgcn_sched_barrier(0);
      DA_MMA();
      __builtin_amdgcn_sched_barrier(0);
      DA_FREAD(cur, 2);
      __builtin_amdgcn_sched_barrier(0);
      DA_MMA2(ga, gb);
      __builtin_amdgcn_sched_barrier(0);
      DA_FREAD2(cur, 3, ga, gb);
      __builtin_amdgcn_sched_barrier(0);
      DA_MMA();
      __builtin_amdgcn_sched_barrier(0);
      dma_wait();
      __syncthreads();
      if (more) DA_FREAD(nxt, 0);
      __builtin_amdgcn_sched_barrier(0);
      DA_MMA2(ga, gb);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
#undef DA_DMA
  } else {
    u32x4_t ra[NCH], rb[NCH];
    constexpr int A_RSTEP = A_KS ? C::NT / (BT / 8) : C::NT / 8;  // tile rows (k rows if k-strided) per chunk
    constexpr int B_RSTEP = B_KS ? C::NT / (BT / 8) : C::NT / 8;
#define DA_GLOAD(kt)                                                                               \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i) {                                              \
      const int r_ = sa.row + i * A_RSTEP;                                                         \
      const bool ok = A_KS ? ((kt) * BK + r_ < dK && m0 + sa.col < d.M)                            \
                           : (m0 + r_ < d.M && (kt) * BK + sa.col < dK);                           \
      const u32x4_t z_ = {0u, 0u, 0u, 0u};                                                         \
      ra[i] = ok ? *reinterpret_cast<const u32x4_t*>(sa.g + i * sa.gstep) : z_;                    \
    }                                                                                              \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i) {                                              \
      const int r_ = sb.row + i * B_RSTEP;                                                         \
      const bool ok = B_KS ? ((kt) * BK + r_ < dK && n0 + sb.col < d.N)                            \
                           : (n0 + r_ < d.N && (kt) * BK + sb.col < dK);                           \
      const u32x4_t z_ = {0u, 0u, 0u, 0u};                                                         \
      rb[i] = ok ? *reinterpret_cast<const u32x4_t*>(sb.g + i * sb.gstep) : z_;                    \
    }                                                                                              \
    sa.g += sa.tstep;                                                                              \
    if (!A_KS && d.a_kwrap && (((kt) + 1) * BK) % d.a_kwrap == 0) sa.g -= d.a_kwrap;               \
    sb.g += sb.tstep;                                                                              \
  } while (0)
#define DA_LSTORE(st)                                                                              \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        *reinterpret_cast<u32x4_t*>((st) + sa.l + i * sa.lstep) = ra[i];                           \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        *reinterpret_cast<u32x4_t*>((st) + A_BYTES + sb.l + i * sb.lstep) = rb[i];                 \
  } while (0)
    DA_GLOAD(0);
    DA_LSTORE(lds);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      char* cur = lds + (kt & 1) * STAGE;
      char* nxt = lds + ((kt + 1) & 1) * STAGE;
      const bool more = kt + 1 < KT;
      if (more) DA_GLOAD(kt + 1);
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        DA_FREAD(cur, ks);
        DA_MMA();
      }
      if (more) DA_LSTORE(nxt);
      __syncthreads();
    }
#undef DA_GLOAD
#undef DA_LSTORE
  }
#undef DA_FREAD
#undef DA_MMA
#undef DA_FREAD2
#undef DA_MMA2
  } else {
  // ---- v_mfma_f32_16x16x32_bf16: a stage is two 32-deep k-steps; per k-step TMI row fragments (two halves H0, H1) and
  // TNJ column fragments.  Read-ahead in registers: while the MFMAs of one half run, the other half's row fragments
  // (and, under H1, the next k-step's column fragments and H0 row fragments) are fetched.
  constexpr int TH = TMI / 2;
  // Measurement builds (-DDA_KLOOP_ABLATE=<bits>, WRONG RESULTS): what the direct-to-LDS loop costs without 1 its
  // fragment reads (the first stage's are kept), 2 its staging loads (after the first two stages), 4 the per-stage
  // wait and barrier, 8 its matrix-core instructions.
  constexpr bool ABL_READ = (DA_KLOOP_ABLATE & 1) != 0, ABL_DMA = (DA_KLOOP_ABLATE & 2) != 0,
                 ABL_BAR = (DA_KLOOP_ABLATE & 4) != 0, ABL_MMA = (DA_KLOOP_ABLATE & 8) != 0;
  bool abl_first = true;
#define DA16_RA(FA, st, ks, h)                                                                     \
  do {                                                                                             \
    if (!(FULL && ABL_READ) || abl_first) {                                                        \
      _Pragma("unroll") for (int i = 0; i < TH; ++i)                                               \
          FA[i] = read_frag16<BT, A_KS>((st), ar0 + ((h) * TH + i) * 16, (ks), lane);              \
    }                                                                                              \
  } while (0)
#define DA16_RB(FB, st, ks)                                                                        \
  do {                                                                                             \
    if (!(FULL && ABL_READ) || abl_first) {                                                        \
      _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                              \
          FB[j] = read_frag16<BT, B_KS>((st) + b_at, br0 + j * 16, (ks), lane);                    \
    }                                                                                              \
  } while (0)
#define DA16_MMA(FA, FB, h)                                                                        \
  do {                                                                                             \
    if (FULL && ABL_MMA) {   /* the fragments are consumed (waited for), nothing is computed */   \
      _Pragma("unroll") for (int i = 0; i < TH; ++i) asm volatile("" ::"v"(FA[i]));               \
      _Pragma("unroll") for (int j = 0; j < TNJ; ++j) asm volatile("" ::"v"(FB[j]));              \
    } else {                                                                                       \
      _Pragma("unroll") for (int i = 0; i < TH; ++i)                                               \
          _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                          \
              acc[(h) * TH + i][j] =                                                               \
                  __builtin_amdgcn_mfma_f32_16x16x32_bf16(FB[j], FA[i], acc[(h) * TH + i][j], 0, 0, 0); \
    }                                                                                              \
  } while (0)
  if (FULL) {
#define DA16_DMA(st)                                                                               \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        dma16(sa.dbase, sa.doff + i * sa.dstep + koff_a, lds_addr(st) + (i * NW + wave) * 1024);   \
    if (b_at != 0) {                                                                               \
      _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                              \
          dma16(sb.dbase, sb.doff + i * sb.dstep + koff_b, lds_addr(st) + A_BYTES + (i * NW + wave) * 1024); \
    }                                                                                              \
    koff_a += (unsigned)(sa.tstep * 2);                                                            \
    if (koff_a == wrap_a) koff_a = 0;                                                              \
    koff_b += (unsigned)(sb.tstep * 2);                                                            \
  } while (0)
    unsigned koff_a = 0, koff_b = 0;
    const unsigned wrap_a = (unsigned)d.a_kwrap * 2u;
    DA16_DMA(lds);
    dma_wait();
    __syncthreads();
    after_first_stage();
    bf16x8_t a0[TH], a1[TH], b0[TNJ], b1[TNJ];
    if (KT > 1) DA16_DMA(lds + STAGE);
    DA16_RB(b0, lds, 0);
    DA16_RA(a0, lds, 0, 0);
    for (int kt = 0; kt < KT; ++kt) {
      char* cur = lds + (kt & 1) * STAGE;
      char* nxt = lds + ((kt + 1) & 1) * STAGE;
      const bool more = kt + 1 < KT;
      DA16_RA(a1, cur, 0, 1);
      __builtin_amdgcn_sched_barrier(0);
      DA16_MMA(a0, b0, 0);
      __builtin_amdgcn_sched_barrier(0);
      DA16_RB(b1, cur, 1);
      DA16_RA(a0, cur, 1, 0);
      __builtin_amdgcn_sched_barrier(0);
      DA16_MMA(a1, b0, 1);
      __builtin_amdgcn_sched_barrier(0);
      DA16_RA(a1, cur, 1, 1);
      __builtin_amdgcn_sched_barrier(0);
      DA16_MMA(a0, b1, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (!ABL_BAR) {
        dma_wait();
        __syncthreads();
      }
      // this stage's buffer is free (every wavefront holds its last fragments): the stage after the next is requested
      // here, a full stage ahead of the barrier that needs it
      if (!ABL_DMA && kt + 2 < KT) DA16_DMA(cur);
      if (more) {
        DA16_RB(b0, nxt, 0);
        DA16_RA(a0, nxt, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      DA16_MMA(a1, b1, 1);
      __builtin_amdgcn_sched_barrier(0);
      abl_first = false;
    }
    if (ABL_BAR) dma_wait();
    __syncthreads();
#undef DA16_DMA
  } else {
    u32x4_t ra[NCH], rb[NCH];
    constexpr int A_RSTEP = A_KS ? C::NT / (BT / 8) : C::NT / 8;
    constexpr int B_RSTEP = B_KS ? C::NT / (BT / 8) : C::NT / 8;
    auto gload = [&](int kt) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int r_ = sa.row + i * A_RSTEP;
        const bool ok = A_KS ? (kt * BK + r_ < dK && m0 + sa.col < d.M) : (m0 + r_ < d.M && kt * BK + sa.col < dK);
        const u32x4_t z_ = {0u, 0u, 0u, 0u};
        ra[i] = ok ? *reinterpret_cast<const u32x4_t*>(sa.g + i * sa.gstep) : z_;
      }
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int r_ = sb.row + i * B_RSTEP;
        const bool ok = B_KS ? (kt * BK + r_ < dK && n0 + sb.col < d.N) : (n0 + r_ < d.N && kt * BK + sb.col < dK);
        const u32x4_t z_ = {0u, 0u, 0u, 0u};
        rb[i] = ok ? *reinterpret_cast<const u32x4_t*>(sb.g + i * sb.gstep) : z_;
      }
      sa.g += sa.tstep;
      if (!A_KS && d.a_kwrap && ((kt + 1) * BK) % d.a_kwrap == 0) sa.g -= d.a_kwrap;   // A again from its first column
      sb.g += sb.tstep;
    };
    auto lstore = [&](char* st) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) *reinterpret_cast<u32x4_t*>(st + sa.l + i * sa.lstep) = ra[i];
#pragma unroll
      for (int i = 0; i < NCH; ++i) *reinterpret_cast<u32x4_t*>(st + A_BYTES + sb.l + i * sb.lstep) = rb[i];
    };
    bf16x8_t a0[TH], a1[TH], b0[TNJ];
    gload(0);
    lstore(lds);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      char* cur = lds + (kt & 1) * STAGE;
      char* nxt = lds + ((kt + 1) & 1) * STAGE;
      const bool more = kt + 1 < KT;
      if (more) gload(kt + 1);
#pragma unroll
      for (int ks = 0; ks < BK / 32; ++ks) {
        DA16_RB(b0, cur, ks);
        DA16_RA(a0, cur, ks, 0);
        DA16_RA(a1, cur, ks, 1);
        DA16_MMA(a0, b0, 0);
        DA16_MMA(a1, b0, 1);
      }
      if (more) lstore(nxt);
      __syncthreads();
    }
  }
#undef DA16_RA
#undef DA16_RB
#undef DA16_MMA
  }
}

template <typename C, bool KS>
__device__ __forceinline__ bf16x8_t read_frag_of(const char* lds, int r0, int ks, int lane) {
  if constexpr (C::MI == 32) return read_frag<C::BT, KS>(lds, r0, ks, lane);
  else return read_frag16<C::BT, KS>(lds, r0, ks, lane);
}
template <typename C>
__device__ __forceinline__ void mma_of(typename C::acc_t& acc, bf16x8_t col, bf16x8_t row) {
  if constexpr (C::MI == 32) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(col, row, acc, 0, 0, 0);
  else acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(col, row, acc, 0, 0, 0);
}

// K loop of one BT x BT tile whose row operand is the SUM of two bf16 matrices of the same layout, formed on the way
// into LDS:  acc += sum_k r_bf16(M + G)(m0 + i, k) * B(n0 + j, k).  The row operand goes through registers (16-byte
// loads of M and of G one stage ahead, eight additions with one rounding each, one 16-byte LDS store per chunk); the
// column operand is k-strided and staged with direct-to-LDS loads as in the DA_LOOP_EDGE form (its ragged dimension
// is kept inside the matrix).  `writeback`: the sums are also stored over M (each element by exactly one tile).
// `any` is or-ed with "some sum is not zero".  M: whole tiles of rows (no checks), dK a multiple of 64.
// Ends with a workgroup barrier; stores of the last stage may still be in flight.
template <typename C, bool A_KS>
__device__ __forceinline__ void gemm_tile_k_loop_sum(typename C::acc_t (&acc)[C::TMI][C::TNJ], const GemmDesc& d, bf16_t* M,
                                                     const bf16_t* G, const bf16_t* B, int dK, int m0, int n0,
                                                     char* lds, int tid, int lane, int wave, int wm, int wn,
                                                     bool writeback, bool& any) {
  constexpr bool B_KS = true;
  constexpr int BT = C::BT, TMI = C::TMI, TNJ = C::TNJ, NCH = C::NCH, NW = C::NT / 64;
  constexpr int A_BYTES = Tile<BT, A_KS>::bytes;
  constexpr int B_BYTES = Tile<BT, B_KS>::bytes;
  constexpr int STAGE = A_BYTES + B_BYTES;
  static_assert(NCH == 4, "the stage barrier's wait count below is written for four stores per stage");
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNJ; ++j)
#pragma unroll
      for (int v = 0; v < C::AV; ++v) acc[i][j][v] = 0.f;

  StageAddr<C, A_KS> sa(M, d.lda, m0, tid, d.M);
  StageAddr<C, B_KS> sb(B, d.ldb, n0, tid, d.N);
  // the thread's chunks as 32-bit byte offsets from the matrix's first element (wave-uniform base + lane offset: the
  // launcher keeps the matrix below 4 GiB)
  const char* const Mc = reinterpret_cast<const char*>(M);
  const char* const Gc = reinterpret_cast<const char*>(G);
  const unsigned gs2 = (unsigned)(sa.gstep * 2), ts2 = (unsigned)(sa.tstep * 2);
  const int ar0 = wm * C::WROWS, br0 = wn * C::WCOLS;
  const int KT = dK / BK;
  bf16x8_t fa[C::MI == 32 ? TMI : TMI / 2], fb[TNJ];
  u32x4_t rm[NCH], rg[NCH];
  unsigned nz = 0u;
  unsigned koff_b = 0;
  unsigned aoff = (unsigned)((sa.g - M) * 2);   // chunk 0 of the stage being loaded

#define DA_SUM_LOAD()                                                                              \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        rm[i] = ldg16(Mc + (size_t)(aoff + i * gs2));                                              \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        rg[i] = ldg16(Gc + (size_t)(aoff + i * gs2));                                              \
  } while (0)
#define DA_SUM_DMA(st)                                                                             \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        dma16(sb.dbase, sb.doff + i * sb.dstep + koff_b, lds_addr(st) + A_BYTES + (i * NW + wave) * 1024); \
    koff_b += (unsigned)(sb.tstep * 2);                                                            \
  } while (0)
// (the stage loaded last: its chunks lie at aoff; the sums go to LDS and, with writeback, over M)
#define DA_SUM_STORE(st)                                                                           \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < NCH; ++i) {                                              \
      u32x4_t o;                                                                                   \
      _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                              \
        const unsigned x = rm[i][q], y = rg[i][q];                                                 \
        o[q] = cvt_pk_bf16(lo_f(x) + lo_f(y), hi_f(x) + hi_f(y));                                  \
        nz |= o[q] & 0x7fff7fffu;                                                                  \
      }                                                                                            \
      *reinterpret_cast<u32x4_t*>((st) + sa.l + i * sa.lstep) = o;                                 \
      if (writeback) stg16(const_cast<char*>(Mc) + (size_t)(aoff + i * gs2), o);                   \
    }                                                                                              \
    aoff += ts2;                                                                                   \
  } while (0)
#define DA_SUM_FREAD(st, ks, FA, FB)                                                               \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        FA[i] = read_frag_of<C, A_KS>((st), ar0 + i * C::MI, (ks), lane);                          \
    _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                                \
        FB[j] = read_frag_of<C, B_KS>((st) + A_BYTES, br0 + j * C::MI, (ks), lane);                \
  } while (0)
#define DA_SUM_MMA(FA, FB)                                                                         \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                            \
            mma_of<C>(acc[i][j], FB[j], FA[i]);                                                    \
  } while (0)

  // (fragments are not double buffered here: the registers hold a stage of M and of G instead, and the loop is
  // bound by the stream of M and G from HBM, not by the matrix cores)
  DA_SUM_LOAD();
  DA_SUM_DMA(lds);
  DA_SUM_STORE(lds);
  dma_wait();
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    char* cur = lds + (kt & 1) * STAGE;
    char* nxt = lds + ((kt + 1) & 1) * STAGE;
    const bool more = kt + 1 < KT;
    if (more) {
      DA_SUM_LOAD();
      DA_SUM_DMA(nxt);
    }
    if constexpr (C::MI == 32) {
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        DA_SUM_FREAD(cur, ks, fa, fb);
        DA_SUM_MMA(fa, fb);
      }
    } else {
      // (16 x 16 blocks: the row fragments of a 32-deep k-step in two halves through the same registers)
#pragma unroll
      for (int ks = 0; ks < BK / 32; ++ks) {
#pragma unroll
        for (int j = 0; j < TNJ; ++j) fb[j] = read_frag16<BT, B_KS>(cur + A_BYTES, br0 + j * 16, ks, lane);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
          for (int i = 0; i < TMI / 2; ++i) fa[i] = read_frag16<BT, A_KS>(cur, ar0 + (h * (TMI / 2) + i) * 16, ks, lane);
#pragma unroll
          for (int i = 0; i < TMI / 2; ++i)
#pragma unroll
            for (int j = 0; j < TNJ; ++j) mma_of<C>(acc[h * (TMI / 2) + i][j], fb[j], fa[i]);
        }
      }
    }
    if (more) DA_SUM_STORE(nxt);
    // the direct-to-LDS loads of the next stage must have landed; the (up to four) stores issued behind them may
    // stay in flight: memory operations of a wavefront complete in the order issued
    if (writeback) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else dma_wait();
    __syncthreads();
  }
  any = any || nz != 0u;
#undef DA_SUM_LOAD
#undef DA_SUM_DMA
#undef DA_SUM_STORE
#undef DA_SUM_FREAD
#undef DA_SUM_MMA
}

}  // namespace
