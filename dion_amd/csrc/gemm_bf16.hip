// Batched bf16 GEMM on the gfx950 matrix cores (v_mfma_f32_16x16x32_bf16, fp32 accumulate; the 32x32x16 form of the
// instruction is kept as a build variant and for GemmDesc::mi32: under the 16x16x32 form the chip holds a 13 % higher
// clock at the same flops per pass, which is worth 3 % to the whole K loop).
//
//   C[b] (M x N) = epilogue( sum_k Aop[b](i,k) * Bop[b](j,k) )
//
// Work decomposition: one workgroup per BT x BT output tile.  Two shapes are built:
//   * BT = 256, 8 wavefronts (2 x 4): each wavefront owns 128 x 64 as 8 x 4 accumulator blocks of
//     16 x 16 (4 x 2 of 32 x 32 in the other form).  Two wavefronts share a SIMD, so while one waits
//     for LDS or a barrier the other keeps the matrix core busy; LDS traffic is 12 fragment reads per
//     32 MFMAs of a 32-deep k-step.
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
#include <atomic>
#include "common.h"
#include "mfma_tile.h"
#include "gemm_bf16_tile.h"
#include <cstdlib>

namespace {

// Kernel argument: up to DA_MAX_GROUPS products; group g owns blocks start[g] .. start[g+1]-1.
struct GemmArgs {
  GemmDesc d[DA_MAX_GROUPS];
  int start[DA_MAX_GROUPS + 1];
  int n;
  int trace;   // 1: every workgroup records its time stamps (measurement hook)
  int diag_k;  // diagonal tiles of a symmetric product stage one panel for both operands when K is at most this
  int interleave;   // bit g: group g's tiles are dealt to the XCDs in turns (see decode_tile)
};

// Which output tile a workgroup owns.  Workgroups are dealt round-robin to the 8 XCDs (each
// with its own L2), so consecutive *logical* tiles -- which share an operand panel -- are
// mapped to the same XCD when the grid divides evenly.
struct TileId { int b, ti, tj; };

template <int BT, bool SYM>
__device__ __forceinline__ TileId decode_tile(const GemmDesc& d, int bid, int nblk, bool xcd_aligned, int interleave) {
  const int tiles_m = (d.M + BT - 1) / BT;
  const int tiles_n = (d.N + BT - 1) / BT;
  const int per_batch = SYM ? tiles_m * (tiles_m + 1) / 2 : tiles_m * tiles_n;
  if (xcd_aligned && (nblk & 7) == 0) {
    // `interleave`: the XCDs take turns at runs of G logical tiles (a super-tile; an eighth of a symmetric matrix), so
    // that all eight work on the same matrix at the same time; otherwise each XCD owns a contiguous eighth of the launch
    const bool sup = !SYM && (((tiles_m % 8) == 0 && (tiles_n % 4) == 0) || ((tiles_m % 4) == 0 && (tiles_n % 8) == 0));
    const int G = sup ? 32 : ((SYM && (per_batch & 7) == 0) ? per_batch >> 3 : 0);
    const int nfull = (interleave && G > 0) ? nblk - nblk % (8 * G) : 0;
    if (bid < nfull) {
      const int xcd = bid & 7, idx = bid >> 3;
      bid = ((idx / G) * 8 + xcd) * G + idx % G;
    } else {   // (the rest of the launch, or all of it: a contiguous eighth per XCD)
      bid = nfull + ((bid - nfull) & 7) * ((nblk - nfull) >> 3) + ((bid - nfull) >> 3);
    }
  }
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
    const int sup_per_row = tiles_n >> 2, sup_rows = tiles_m >> 3;
    int sr, sc;
    // (dealt in turns, the eight XCDs then cover whole columns of super-tiles: a B panel is in use by all the XCDs
    // that need it at the same time)
    if (interleave) { sc = sup / sup_rows; sr = sup - sc * sup_rows; }
    else { sr = sup / sup_per_row; sc = sup - sr * sup_per_row; }
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
constexpr int DA_TRACE_TILES = 65536;
constexpr int DA_TRACE_WORDS = 6;
__device__ unsigned long long da_tile_trace[DA_TRACE_WORDS * DA_TRACE_TILES];
std::atomic<bool> g_tile_trace{false};

template <typename C, bool A_KS, bool B_KS, bool SYM, int MODE>
__global__ __launch_bounds__(C::NT) void gemm_bf16_kernel(GemmArgs args) {
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
  constexpr int BT = C::BT, TMI = C::TMI, TNJ = C::TNJ;
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = wave_uniform(tid >> 6);
  const int wm = wave / C::WGN, wn = wave % C::WGN;
  const TileId tile = decode_tile<BT, SYM>(d, (int)blockIdx.x - blk0, args.start[grp + 1] - blk0, (blk0 & 7) == 0, (args.interleave >> grp) & 1);
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

  typename C::acc_t acc[TMI][TNJ];
  gemm_tile_k_loop<C, A_KS, B_KS, MODE>(acc, d, A, B, dK, m0, n0, lds, tid, lane, wave, wm, wn, DaNoHook(),
                                        SYM && ti == tj && A == B && dK <= args.diag_k);
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

// dion_amd_set_option("edge_loop"): -1 the environment decides (DION_AMD_NO_EDGE_LOOP), 0 ragged products take the
// bounds-checked K loop, 1 the direct-to-LDS loop with edge tiles where it applies.
std::atomic<int> g_opt_edge_loop{-1};

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
  static const bool edge_env = [] { const char* e = getenv("DION_AMD_NO_EDGE_LOOP"); return !(e && atoi(e)); }();
  const int edge_opt = g_opt_edge_loop.load(std::memory_order_relaxed);
  const bool edge_on = edge_opt >= 0 ? edge_opt != 0 : edge_env;
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
  // A diagonal tile that stages one panel runs ahead of the tiles it shares that panel with.  In a launch of a few
  // rounds that shortens the tail (Llama-8B layer: X X^T 0.81 -> 0.77 ms); over many rounds of a long K the tiles
  // lose each other in the L2 (32 x 4096 x 14336: 1.7 x the fetched bytes, 6.93 -> 7.35 ms), so there only up to
  // K = 4096 (bA + cAA: 2 % faster with it).  DION_AMD_DIAG_K overrides the limit (0: never).
  // With a contiguous eighth of the launch per XCD the eight XCDs work on eight different matrices.  A launch whose
  // operands exceed the 256 MB Infinity Cache has the XCDs take turns at the tiles of one matrix instead: a panel then
  // comes from HBM once and for the other XCDs from that cache (32 x 4096 x 14336: X' = aX + BX 13.5 -> 13.0 ms,
  // X X^T 7.0 -> 6.8 ms; all Newton-Schulz products of Llama-3-8B 443 -> 437 ms per step; launches of a few matrices
  // are up to 1 % faster without).  DION_AMD_XCD_INTERLEAVE=0|1 overrides the rule.
  static const int il_env = [] { const char* e = getenv("DION_AMD_XCD_INTERLEAVE"); return e ? atoi(e) : -1; }();
  args.interleave = 0;
  for (int g = 0; g < n; ++g) {
    const double bytes = 2.0 * d[g].batch * ((double)d[g].M * d[g].K + (SYM ? 0.0 : (double)d[g].N * d[g].K));
    if (il_env >= 0 ? il_env != 0 : bytes > 512.0 * 1048576.0) args.interleave |= 1 << g;
  }
  static const int diag_k_env = [] { const char* e = getenv("DION_AMD_DIAG_K"); return e ? atoi(e) : -1; }();
  args.diag_k = diag_k_env >= 0 ? diag_k_env : (blocks <= 4LL * da_cu_count() ? 0x7fffffff : 4096);
  for (int g = 0; g < n; ++g)   // the weight-update epilogue exists for interior tiles of plain bf16 AXPBY products
    if (d[g].upd_tab && (!full || SYM || d[g].c_dtype != DA_BF16 || d[g].epilogue != DA_EPI_AXPBY)) return DA_ERR_ARG;
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
typedef Cfg<256, 2, 4, 32> Big32;      // (GemmDesc::mi32)
typedef Cfg<128, 2, 2, 32> Small32;

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
        a.epilogue != f.epilogue || a.c_dtype != f.c_dtype || a.faithful != f.faithful || (a.mi32 != 0) != (f.mi32 != 0))
      return DA_ERR_ARG;
    if (a.mi32 && (a.symmetric || a.a_kstrided || a.b_kstrided)) return DA_ERR_ARG;
    // insertion sort, longest K first: long tiles start early, short ones fill the tail
    int pos = g;
    while (pos > 0 && d[pos - 1].K < a.K) { d[pos] = d[pos - 1]; --pos; }
    d[pos] = a;
  }
  if (d[0].mi32) {
    if (choose_tile(d, n) == 256) return launch<Big32, false, false, false>(d, n, stream);
    return launch<Small32, false, false, false>(d, n, stream);
  }
  if (choose_tile(d, n) == 256) return dispatch_layout<Big>(d, n, stream);
  return dispatch_layout<Small>(d, n, stream);
}

void da_gemm_bf16_set_edge_loop(int v) { g_opt_edge_loop.store(v < 0 ? -1 : (v != 0), std::memory_order_relaxed); }

// What the launcher would do with one product of these dimensions, without launching anything:
// tile edge (128 or 256), plus 1 if the K loop is the direct-to-LDS one.
int da_gemm_bf16_plan(const GemmDesc& d) {
  const int bt = choose_tile(&d, 1);
  return bt + (all_interior(&d, 1, bt) ? 1 : 0);
}

int da_gemm_bf16(const GemmDesc& d, hipStream_t stream) { return da_gemm_bf16_grouped(&d, 1, stream); }

// Whether the grouped launch of these products runs the interior (direct-to-LDS, unchecked) form for every tile:
// the form the weight-update epilogue (GemmDesc::upd_tab) exists in.
bool da_gemm_bf16_all_interior(const GemmDesc* d, int n) {
  if (!d || n <= 0 || n > DA_MAX_GROUPS) return false;
  return all_interior(d, n, choose_tile(d, n));
}

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
