// Batched bf16 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate).
//
//   C[b] (M x N) = epilogue( sum_k Aop[b](i,k) * Bop[b](j,k) )
//
// Work decomposition: one workgroup per BT x BT output tile.  Two shapes are built:
//   * BT = 256, 8 wavefronts (2 x 4): each wavefront owns 128 x 64 as 4 x 2 accumulators of
//     32 x 32.  Two wavefronts share a SIMD, so while one waits for LDS or a barrier the
//     other keeps the matrix core busy; LDS traffic is 6 fragment reads per 8 MFMAs.
//   * BT = 128, 4 wavefronts (2 x 2), 64 x 64 each: for problems too small to fill the
//     256 CUs with large tiles.
// The K loop advances 64 elements per stage and is double buffered through LDS.
//
// Operand staging in LDS:
//   * k-contiguous operand (rows x K in memory): tile [BT][64] of 16-byte chunks, chunk
//     index XOR-swizzled with ((row >> 1) & 7): the 16 lanes served per clock by a
//     ds_read_b128 fragment read (16 consecutive rows, same logical chunk) then fall into
//     16 different 16-byte slots of the 64-bank, 256-byte LDS line.
//   * k-strided operand (K x rows in memory, e.g. X in  X' = aX + B X): the tile keeps the
//     memory orientation, [64][BT] with 32-byte slots XOR-swizzled by (k-row & 3), and the
//     fragment is fetched with two ds_read_b64_tr_b16 (the LDS transpose read of CDNA4),
//     which hands each lane the four k-consecutive values of its own column.  No register
//     shuffles, no second copy of X.
// Interior tiles are staged with direct-to-LDS loads (global_load_lds_dwordx4): no staging
// registers and no ds_write instructions; the swizzles are applied to the global address.
//
// The MFMA is issued with the operands swapped (D' = Bfrag x Afrag^T), so that a lane ends
// up with four *column-consecutive* results of one output row; the epilogue then passes the
// accumulators through LDS so that C and E move as 16-byte row segments.  For a symmetric
// result only tiles on or above the diagonal are computed and every off-diagonal tile is
// also written transposed.
#include "common.h"
#include "mfma_tile.h"
#include <cstdlib>

namespace {

// Kernel argument: up to DA_MAX_GROUPS products; group g owns blocks start[g] .. start[g+1]-1.
struct GemmArgs {
  GemmDesc d[DA_MAX_GROUPS];
  int start[DA_MAX_GROUPS + 1];
  int n;
  int trace;   // 1: every workgroup records its time stamps (measurement hook)
};

template <int BT_, int WGM_, int WGN_>
struct Cfg {
  static constexpr int BT = BT_, WGM = WGM_, WGN = WGN_;
  static constexpr int NT = 64 * WGM * WGN;        // threads
  static constexpr int TMI = BT / (32 * WGM);      // accumulators per wavefront, row direction
  static constexpr int TNJ = BT / (32 * WGN);      // ... column direction
  static constexpr int NCH = BT * 8 / NT;          // 16-byte chunks per thread per operand stage
  static constexpr int WROWS = BT / WGM, WCOLS = BT / WGN;
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

// Which output tile a workgroup owns.  Workgroups are dealt round-robin to the 8 XCDs (each
// with its own L2), so consecutive *logical* tiles -- which share an operand panel -- are
// mapped to the same XCD when the grid divides evenly.
struct TileId { int b, ti, tj; };

template <int BT, bool SYM>
__device__ __forceinline__ TileId decode_tile(const GemmDesc& d, int bid, int nblk, bool xcd_aligned) {
  const int tiles_m = (d.M + BT - 1) / BT;
  const int tiles_n = (d.N + BT - 1) / BT;
  const int per_batch = SYM ? tiles_m * (tiles_m + 1) / 2 : tiles_m * tiles_n;
  if (xcd_aligned && (nblk & 7) == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);
  TileId r;
  r.b = bid / per_batch;
  int t = bid - r.b * per_batch;
  if (SYM) {
    r.ti = 0;
    int len = tiles_m;
    while (t >= len) { t -= len; ++r.ti; --len; }
    r.tj = r.ti + t;
  } else if ((tiles_m % 8) == 0 && (tiles_n % 4) == 0) {
    // 8 x 4 super-tiles: the 32 workgroups that an XCD runs at a time then share 8 A panels and
    // 4 B panels (12 panel loads per k-step instead of 33 for a row of 32 tiles); measured 3-7 %
    // faster than row-major order on 4096 x 14336, and a little better than 4 x 8
    const int sup = t >> 5, within = t & 31;
    const int sup_per_row = tiles_n >> 2;
    const int sr = sup / sup_per_row, sc = sup - sr * sup_per_row;
    r.ti = sr * 8 + (within >> 2);
    r.tj = sc * 4 + (within & 3);
  } else if ((tiles_m % 4) == 0 && (tiles_n % 8) == 0) {
    const int sup = t >> 5, within = t & 31;
    const int sup_per_row = tiles_n >> 3;
    const int sr = sup / sup_per_row, sc = sup - sr * sup_per_row;
    r.ti = sr * 4 + (within >> 3);
    r.tj = sc * 8 + (within & 7);
  } else {
    r.ti = t / tiles_n;
    r.tj = t - r.ti * tiles_n;
  }
  return r;
}

// The accumulators go through LDS (the stage buffers are free by now), one 32-row band of the
// wavefront's sub-tile at a time, so that C and E move as 16-byte row segments.  Each wavefront
// stages through its own LDS region, so only wavefront-level ordering is needed inside.
// Output dtype, epilogue form and rounding mode are compile-time here: evaluated per element at
// run time they cost more than the MFMAs of a short-K product.
template <typename C, bool SYM, bool FULL, bool CF32, bool HAS_E, bool FAITHFUL, bool S1_ONE>
__device__ __forceinline__ void epilogue_impl(f32x16_t (&acc)[C::TMI][C::TNJ], const GemmDesc& d, char* lds, int b,
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
  // E is requested up to three bands ahead (registers that the K loop's fragments no longer need), so that a
  // tile's epilogue pays one memory latency and not one per band; an fp32 E (twice the registers) one band ahead.
  constexpr int DEPTH = (!HAS_E || CF32) ? 1 : (C::TMI < 3 ? C::TMI : 3);
  u32x4_t ev[DEPTH][NPASS][NV];
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
  for (int i = 0; i < C::TMI; ++i) {
    {
      float* row = stg + (lane & 31) * PITCH + (lane >> 5) * 4;
#pragma unroll
      for (int j = 0; j < C::TNJ; ++j)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq)
          *reinterpret_cast<float4*>(row + j * 32 + vq * 8) =
              make_float4(acc[i][j][vq * 4], acc[i][j][vq * 4 + 1], acc[i][j][vq * 4 + 2], acc[i][j][vq * 4 + 3]);
    }
    wave_sync_lds();
    const int band_m = wm0 + i * 32;
    u32x4_t ec[NPASS][NV];
    if (HAS_E) {
#pragma unroll
      for (int pass = 0; pass < NPASS; ++pass)
#pragma unroll
        for (int h = 0; h < NV; ++h) ec[pass][h] = ev[i % DEPTH][pass][h];
      if (i + DEPTH < C::TMI) load_e(i + DEPTH, ev[i % DEPTH]);
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
          stg16(Cp, pk);
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
__device__ __forceinline__ void epilogue(f32x16_t (&acc)[C::TMI][C::TNJ], const GemmDesc& d, char* lds, int b, int ti,
                                         int tj, int m0, int n0, int wave, int lane, int wm, int wn) {
  const bool mirror = SYM && (ti != tj);
  const bool cf32 = d.c_dtype == DA_F32, has_e = d.epilogue == DA_EPI_AXPBY, fa = d.faithful != 0;
  const bool one = d.s1 == 1.f;   // rounding-faithful bf16 output: the exact multiplication by 1 is left out
#define DA_EPI(CF, HE, FA, S1) \
  epilogue_impl<C, SYM, FULL, CF, HE, FA, S1>(acc, d, lds, b, mirror, m0, n0, wave, lane, wm, wn)
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
}

// ---------------------------------------------------------------------------------------
// One kernel, two K loops, three modes.
//   DA_LOOP_INTERIOR: every tile is interior (M, N multiples of BT, K a multiple of 64).  Stages are
//     fetched with direct-to-LDS loads issued one stage ahead; the only wait is the
//     vmcnt(0) in front of the per-stage barrier.  No bounds checks anywhere.
//   DA_LOOP_EDGE: the same K loop for products whose ragged dimension belongs to a k-strided operand (its chunks
//     are kept inside the matrix) and whose other operand has whole tiles; the epilogue checks bounds.  Dion's
//     rank-r products at a rank that is not a multiple of the tile edge (r = 192).
//   DA_LOOP_CHECKED: bounds-checked 16-byte loads into registers (out-of-range chunks zero filled),
//     written to LDS after the stage's MFMAs.
// ---------------------------------------------------------------------------------------
// Measurement hook: per workgroup (tile) of the last traced launch, the 100 MHz counter at the start, after the
// K loop and at the end, the hardware id of the CU it ran on, and the shader-clock counter at the start and the end.
constexpr int DA_LOOP_CHECKED = 0, DA_LOOP_INTERIOR = 1, DA_LOOP_EDGE = 2;
constexpr int DA_TRACE_TILES = 65536;
constexpr int DA_TRACE_WORDS = 6;
__device__ unsigned long long da_tile_trace[DA_TRACE_WORDS * DA_TRACE_TILES];
std::atomic<bool> g_tile_trace{false};

template <typename C, bool A_KS, bool B_KS, bool SYM, int MODE>
__global__ __launch_bounds__(C::NT) void gemm_bf16_kernel(GemmArgs args) {
  constexpr bool FULL = MODE != DA_LOOP_CHECKED;   // the direct-to-LDS K loop
  const bool trace = args.trace && blockIdx.x < DA_TRACE_TILES;
  unsigned long long ts0 = 0, ts1 = 0, tc0 = 0;
  if (trace) {
    ts0 = __builtin_amdgcn_s_memrealtime();
    tc0 = __builtin_amdgcn_s_memtime();
  }
  // which of the grouped products this workgroup belongs to (groups own contiguous block ranges)
  int grp = 0;
#pragma unroll
  for (int q = 1; q < DA_MAX_GROUPS; ++q)
    if (q < args.n && (int)blockIdx.x >= args.start[q]) grp = q;
  const GemmDesc& d = args.d[grp];
  const int blk0 = args.start[grp];
  constexpr int BT = C::BT, TMI = C::TMI, TNJ = C::TNJ, NCH = C::NCH, NW = C::NT / 64;
  constexpr int A_BYTES = Tile<BT, A_KS>::bytes;
  constexpr int B_BYTES = Tile<BT, B_KS>::bytes;
  constexpr int STAGE = A_BYTES + B_BYTES;
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = wave_uniform(tid >> 6);
  const int wm = wave / C::WGN, wn = wave % C::WGN;
  const TileId tile = decode_tile<BT, SYM>(d, (int)blockIdx.x - blk0, args.start[grp + 1] - blk0, (blk0 & 7) == 0);
  const int ti = tile.ti, tj = tile.tj;
  // with K slices the tile index counts (slice, matrix) pairs: the slice's partial product is matrix tile.b of C
  int b = tile.b, dK = d.K;
  long long k0 = 0;
  if (d.k_slices > 1) {
    const int slice = tile.b / d.batch;
    b = tile.b - slice * d.batch;
    k0 = (long long)slice * d.k_slice;
    dK = d.K - (int)k0 < d.k_slice ? d.K - (int)k0 : d.k_slice;
  }
  if (d.gate && (d.gate[b] != 0) != (d.gate_want != 0)) return;   // (before any barrier: the whole workgroup leaves)
  const int m0 = ti * BT, n0 = tj * BT;
  const bf16_t* A = (d.Atab ? static_cast<const bf16_t*>(d.Atab[b]) + d.a_off : static_cast<const bf16_t*>(d.A) + (long long)b * d.sA) +
                    k0 * (A_KS ? d.lda : 1);
  const bf16_t* B = (d.Btab ? static_cast<const bf16_t*>(d.Btab[b]) : static_cast<const bf16_t*>(d.B) + (long long)b * d.sB) +
                    k0 * (B_KS ? d.ldb : 1);

  f32x16_t acc[TMI][TNJ];
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  StageAddr<C, A_KS> sa(A, d.lda, m0, tid, d.M);
  StageAddr<C, B_KS> sb(B, d.ldb, n0, tid, d.N);
  const int ar0 = wm * C::WROWS, br0 = wn * C::WCOLS;
  const int KT = (dK + BK - 1) / BK;
  bf16x8_t fa[TMI], fb[TNJ];

#define DA_FREAD(st, ks)                                                                           \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        fa[i] = read_frag<BT, A_KS>((st), ar0 + i * 32, (ks), lane);                               \
    _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                                \
        fb[j] = read_frag<BT, B_KS>((st) + A_BYTES, br0 + j * 32, (ks), lane);                     \
  } while (0)
#define DA_FREAD2(st, ks, FA, FB)                                                                  \
  do {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TMI; ++i)                                                \
        FA[i] = read_frag<BT, A_KS>((st), ar0 + i * 32, (ks), lane);                               \
    _Pragma("unroll") for (int j = 0; j < TNJ; ++j)                                                \
        FB[j] = read_frag<BT, B_KS>((st) + A_BYTES, br0 + j * 32, (ks), lane);                     \
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
    _Pragma("unroll") for (int i = 0; i < NCH; ++i)                                                \
        dma16(sb.dbase, sb.doff + i * sb.dstep + koff_b, lds_addr(st) + A_BYTES + (i * NW + wave) * 1024); \
    koff_a += (unsigned)(sa.tstep * 2);                                                            \
    if (koff_a == wrap_a) koff_a = 0;                                                              \
    koff_b += (unsigned)(sb.tstep * 2);                                                            \
  } while (0)
    unsigned koff_a = 0, koff_b = 0;   // byte offset of the stage within the operand (< 4 GiB: checked by the launcher)
    const unsigned wrap_a = (unsigned)d.a_kwrap * 2u;   // A read again from its first column (0: never, koff_a > 0 here)
    DA_DMA(lds);
    dma_wait();
    __syncthreads();
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
  if (trace) ts1 = __builtin_amdgcn_s_memrealtime();
  epilogue<C, SYM, MODE == DA_LOOP_INTERIOR>(acc, d, lds, tile.b, ti, tj, m0, n0, wave, lane, wm, wn);
  if (trace) {
    __syncthreads();
    if (tid == 0) {
      const unsigned hw = __builtin_amdgcn_s_getreg(4 | (31 << 11));      // HW_ID: CU, shader array, shader engine
      const unsigned xcc = __builtin_amdgcn_s_getreg(20 | (3 << 11));     // XCC_ID
      unsigned long long* t = da_tile_trace + DA_TRACE_WORDS * (size_t)blockIdx.x;
      t[0] = ts0; t[1] = ts1; t[2] = __builtin_amdgcn_s_memrealtime();
      t[3] = ((unsigned long long)xcc << 32) | hw;
      t[4] = tc0; t[5] = __builtin_amdgcn_s_memtime();
    }
  }
}

// Bytes from the first to the last element a workgroup reads of one operand (BT rows, all of K).
long long da_tile_span_bytes(bool kstrided, int bt, long long ld, long long K) {
  return 2 * (kstrided ? (K - 1) * ld + bt : (bt - 1) * ld + K);
}

// Whether every tile of every group is interior for tile edge `bt` (the direct-to-LDS K loop).  That path
// addresses a tile's operands with 32-bit byte offsets from the tile's first element: an operand whose tile
// spans 4 GiB or more takes the register-staged path, which walks 64-bit pointers.
bool all_interior(const GemmDesc* d, int n, int bt) {
  for (int g = 0; g < n; ++g) {
    if (d[g].M % bt || d[g].N % bt || d[g].K % BK) return false;
    if (da_tile_span_bytes(d[g].a_kstrided != 0, bt, d[g].lda, d[g].K) >= (1LL << 32)) return false;
    if (da_tile_span_bytes(d[g].b_kstrided != 0, bt, d[g].ldb, d[g].K) >= (1LL << 32)) return false;
  }
  return true;
}

// Whether the direct-to-LDS K loop can run with edge tiles: K whole stages, every k-contiguous operand in whole
// tiles (its rows are fetched unconditionally), every k-strided operand at least one chunk wide (multiples of 8
// by the alignment contract), 32-bit offsets as above.
bool edge_loop_ok(const GemmDesc* d, int n, int bt) {
  for (int g = 0; g < n; ++g) {
    if (d[g].K % BK) return false;
    if (!d[g].a_kstrided && d[g].M % bt) return false;
    if (!d[g].b_kstrided && d[g].N % bt) return false;
    if (d[g].a_kstrided && (d[g].M < 8 || d[g].M % 8)) return false;
    if (d[g].b_kstrided && (d[g].N < 8 || d[g].N % 8)) return false;
    if (da_tile_span_bytes(d[g].a_kstrided != 0, bt, d[g].lda, d[g].K) >= (1LL << 32)) return false;
    if (da_tile_span_bytes(d[g].b_kstrided != 0, bt, d[g].ldb, d[g].K) >= (1LL << 32)) return false;
  }
  return true;
}

template <typename C>
long long tiles_of(const GemmDesc& d) {
  const long long tm = (d.M + C::BT - 1) / C::BT, tn = (d.N + C::BT - 1) / C::BT;
  return (d.symmetric ? tm * (tm + 1) / 2 : tm * tn) * d.batch * (d.k_slices > 1 ? d.k_slices : 1);
}

template <typename C, bool A_KS, bool B_KS, bool SYM>
int launch(const GemmDesc* d, int n, hipStream_t stream) {
  constexpr int BT = C::BT;
  constexpr int stage2 = 2 * (Tile<BT, A_KS>::bytes + Tile<BT, B_KS>::bytes);
  constexpr int epi = (C::NT / 64) * 32 * (C::WCOLS + 4) * 4;
  constexpr int smem = stage2 > epi ? stage2 : epi;
  auto kfull = gemm_bf16_kernel<C, A_KS, B_KS, SYM, DA_LOOP_INTERIOR>;
  auto kedge = gemm_bf16_kernel<C, A_KS, B_KS, SYM, (A_KS || B_KS) && !SYM ? DA_LOOP_EDGE : DA_LOOP_CHECKED>;
  auto kgen = gemm_bf16_kernel<C, A_KS, B_KS, SYM, DA_LOOP_CHECKED>;
  static DaOncePerDevice configured;
  const int rc_cfg = configured.run([&]() -> int {
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kfull), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kedge), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kgen), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return DA_OK;
  });
  if (rc_cfg) return rc_cfg;
  GemmArgs args{};
  args.n = n;
  args.trace = g_tile_trace.load(std::memory_order_relaxed) ? 1 : 0;
  const bool full = all_interior(d, n, BT);
  static const bool edge_on = [] { const char* e = getenv("DION_AMD_NO_EDGE_LOOP"); return !(e && atoi(e)); }();
  const bool edge = !full && edge_on && (A_KS || B_KS) && !SYM && edge_loop_ok(d, n, BT);
  long long blocks = 0;
  for (int g = 0; g < n; ++g) {
    args.d[g] = d[g];
    args.start[g] = (int)blocks;
    const long long t = tiles_of<C>(d[g]);
    if (t <= 0) return DA_ERR_LIMIT;
    blocks += t;
    if (blocks > 0x7fffffffLL) return DA_ERR_LIMIT;
  }
  for (int g = n; g <= DA_MAX_GROUPS; ++g) args.start[g] = (int)blocks;
  if (!full && !edge)   // the bounds-checked K loop walks A with a pointer: no wrap-around there
    for (int g = 0; g < n; ++g)
      if (d[g].a_kwrap) return DA_ERR_ARG;
  hipLaunchKernelGGL(full ? kfull : (edge ? kedge : kgen), dim3((unsigned)blocks), dim3(C::NT), smem, stream, args);
  return da_launch_status();
}

template <typename C>
int dispatch_layout(const GemmDesc* d, int n, hipStream_t stream) {
  const GemmDesc& f = d[0];
  if (f.symmetric) return launch<C, false, false, true>(d, n, stream);
  if (!f.a_kstrided && !f.b_kstrided) return launch<C, false, false, false>(d, n, stream);
  if (!f.a_kstrided && f.b_kstrided) return launch<C, false, true, false>(d, n, stream);
  if (f.a_kstrided && !f.b_kstrided) return launch<C, true, false, false>(d, n, stream);
  return launch<C, true, true, false>(d, n, stream);
}

int check_desc(const GemmDesc& d) {
  if ((!d.A && !d.Atab) || (!d.B && !d.Btab) || (!d.C && !d.Ctab) || d.M <= 0 || d.N <= 0 || d.K <= 0 || d.batch <= 0)
    return DA_ERR_ARG;
  if (d.epilogue == DA_EPI_AXPBY && !d.E && !d.Etab) return DA_ERR_ARG;
  if (d.c_dtype != DA_BF16 && d.c_dtype != DA_F32) return DA_ERR_DTYPE;
  if ((d.K | d.N | d.lda | d.ldb | d.ldc) & 7) return DA_ERR_ALIGN;
  if ((d.sA | d.sB | d.sC | d.a_off) & 7) return DA_ERR_ALIGN;
  if (d.a_off && !d.Atab) return DA_ERR_ARG;
  if ((d.E || d.Etab) && ((d.lde & 7) || (d.sE & 7))) return DA_ERR_ALIGN;
  if (d.a_kstrided && (d.M & 7)) return DA_ERR_ALIGN;
  if (((uintptr_t)d.A | (uintptr_t)d.B | (uintptr_t)d.C | (uintptr_t)d.E) & 15) return DA_ERR_ALIGN;
  if (d.symmetric && (d.M != d.N || d.a_kstrided || d.b_kstrided)) return DA_ERR_ARG;
  if (d.a_kwrap && (d.a_kwrap < 0 || d.a_kstrided || d.a_kwrap % BK || d.K % d.a_kwrap)) return DA_ERR_ARG;
  if (d.c2_off && (d.c_dtype != DA_BF16 || d.epilogue != DA_EPI_STORE || d.faithful || d.symmetric || (d.c2_off & 7)))
    return DA_ERR_ARG;
  if (d.k_slices < 0 || (d.k_slices > 1 && (d.k_slice <= 0 || d.k_slice % BK || (long long)(d.k_slices - 1) * d.k_slice >= d.K ||
                                            (long long)d.k_slices * d.k_slice < d.K || d.c_dtype != DA_F32 ||
                                            d.epilogue != DA_EPI_STORE || d.Ctab || d.a_kwrap || d.c2_off || d.symmetric)))
    return DA_ERR_ARG;
  return DA_OK;
}

// Estimated duration of the launch with tile configuration C, in units of "one 64-deep stage of a
// 256 x 256 tile on a whole CU": groups are taken longest-K first (the order they are launched
// in), `slots` tiles run at a time, the last group's partial round is rounded up, and no launch
// is shorter than its longest tile.
template <typename C>
double launch_cost(const GemmDesc* d, int n, int slots, double unit) {
  double level = 0.0, longest = 0.0;
  for (int g = 0; g < n; ++g) {
    const double kt = (double)(((d[g].k_slices > 1 ? d[g].k_slice : d[g].K) + BK - 1) / BK);
    const double rounds = (double)tiles_of<C>(d[g]) / slots;
    if (g + 1 < n) {
      level += rounds * kt;
    } else {
      // the last group first fills what the earlier ones left of their final round
      const double frac = level > 0.0 ? 0.5 : 0.0;
      double r = rounds - frac;
      if (r < 0.0) r = 0.0;
      level += ((double)(long long)(r + 0.999999)) * kt;
    }
    if (kt > longest) longest = kt;
  }
  return unit * (level > longest ? level : longest);
}

typedef Cfg<256, 2, 4> Big;
typedef Cfg<128, 2, 2> Small;

// Tile choice by cost model: 256 x 256 tiles run one per CU, 128 x 128 tiles two per CU; a small
// tile does a quarter of the work on half a CU at about 2/3 of the large tile's MFMA efficiency
// (measured on grouped Newton-Schulz products of 768-wide matrices).
// Interior-only (direct-to-LDS) eligibility wins over either.
int choose_tile(const GemmDesc* d, int n) {
  static const int forced = [] { const char* e = getenv("DION_AMD_TILE"); return e ? atoi(e) : 0; }();
  if (forced == 128 || forced == 256) return forced;
  bool fits_big = true;
  // (a 192-wide product fills three quarters of a 256-tile: still cheaper than one and a half 128-tiles -- rank-192
  // P = BQ 34 -> 29.5 us per GPT-small bucket)
  for (int g = 0; g < n; ++g) fits_big = fits_big && d[g].M >= 192 && d[g].N >= 192;
  // (either form of the direct-to-LDS K loop counts)
  const bool may_edge = !d[0].symmetric && (d[0].a_kstrided || d[0].b_kstrided);
  const bool full_big = all_interior(d, n, 256) || (may_edge && edge_loop_ok(d, n, 256));
  const bool full_small = all_interior(d, n, 128) || (may_edge && edge_loop_ok(d, n, 128));
  const double cost_big = launch_cost<Big>(d, n, 256, 4.0);
  const double cost_small = launch_cost<Small>(d, n, 512, 3.0);
  return fits_big && (full_big || !full_small) && cost_big <= cost_small ? 256 : 128;
}

}  // namespace

// Alignment contract: K, N, every leading dimension and every batch stride are multiples
// of 8 elements (16-byte chunks); M too when A is k-strided; pointers 16-byte aligned.
int da_gemm_bf16_grouped(const GemmDesc* din, int n, hipStream_t stream) {
  if (!din || n <= 0 || n > DA_MAX_GROUPS) return DA_ERR_ARG;
  GemmDesc d[DA_MAX_GROUPS];
  for (int g = 0; g < n; ++g) {
    const int rc = check_desc(din[g]);
    if (rc) return rc;
    const GemmDesc &a = din[g], &f = din[0];
    if (a.symmetric != f.symmetric || a.a_kstrided != f.a_kstrided || a.b_kstrided != f.b_kstrided ||
        a.epilogue != f.epilogue || a.c_dtype != f.c_dtype || a.faithful != f.faithful)
      return DA_ERR_ARG;
    // insertion sort, longest K first: long tiles start early, short ones fill the tail
    int pos = g;
    while (pos > 0 && d[pos - 1].K < a.K) { d[pos] = d[pos - 1]; --pos; }
    d[pos] = a;
  }
  if (choose_tile(d, n) == 256) return dispatch_layout<Big>(d, n, stream);
  return dispatch_layout<Small>(d, n, stream);
}

// What the launcher would do with one product of these dimensions, without launching anything:
// tile edge (128 or 256), plus 1 if the K loop is the direct-to-LDS one.
int da_gemm_bf16_plan(const GemmDesc& d) {
  const int bt = choose_tile(&d, 1);
  return bt + (all_interior(&d, 1, bt) ? 1 : 0);
}

int da_gemm_bf16(const GemmDesc& d, hipStream_t stream) { return da_gemm_bf16_grouped(&d, 1, stream); }

// ---- measurement hook: time stamps of the tiles of the bf16 GEMM launches (see include/dion_amd.h)
extern "C" int dion_amd_tile_trace_enable(int on) {
  g_tile_trace.store(on != 0, std::memory_order_relaxed);
  return DA_OK;
}
extern "C" int dion_amd_tile_trace_read(void* dst, int tiles) {
  if (!dst || tiles <= 0 || tiles > DA_TRACE_TILES) return DA_ERR_ARG;
  DA_HIP_CHECK(hipDeviceSynchronize());
  DA_HIP_CHECK(hipMemcpyFromSymbol(dst, HIP_SYMBOL(da_tile_trace), (size_t)tiles * DA_TRACE_WORDS * sizeof(unsigned long long)));
  return DA_OK;
}
