// Dion's error feedback and weight update as ONE pass over the momentum and the weights (bf16 factors):
//
//   M <- M - (1 - mu) P R^T        X <- (1 - lr wd) X - lr' P Qn^T          (reference dion/dion.py:851-872, 1494-1530)
//
// Both are rank-r products of the same P; with r = 512 their arithmetic intensity (244 flop per byte of M and X
// moved) sits next to the machine balance, so neither the matrix cores nor HBM may idle while the other works.
// A workgroup that computes a tile and then writes it does exactly that: K loop (MFMA-bound), then epilogue
// (HBM-bound).  Here a persistent workgroup holds TWO groups of four wavefronts (one wavefront of each group
// per SIMD) that take turns: while group A runs the K loop of its 128 x 128 tile -- two accumulator sets fed
// from one P fragment, P R^T and P Qn^T -- group B reads M and X of its previous tile, applies the two
// rounding-faithful updates and writes them back; then they swap.  The matrix cores see one K loop after the
// other with no epilogue in between, and the M / X traffic of a tile is spread over the K loop of the next.
//
// Synchronisation is the workgroup barrier only: a slot (one tile's K loop) has one barrier per 64-deep stage,
// and the group that is not in its K loop executes the same number of barriers between the pieces of its
// epilogue (8 pieces of 16 rows x 64 columns per wavefront and output).  The stage ring (2 x 48 KB: P, R and Qn
// tiles, filled by direct-to-LDS loads) is shared: only one group is in a K loop at a time, and it also requests the
// first stage of the other group's next tile during its own last stage, so the epilogue group never waits for a
// load it has not asked for.
#include "dion.h"
#include "mfma_tile.h"
#include <cstdlib>

namespace {

constexpr int FT = 128;                  // tile edge (rows of P, rows of R / Qn)
constexpr int OPND = FT * BK * 2;        // one operand tile of a stage: 128 rows x 64 k of bf16
constexpr int STAGE = 3 * OPND;          // P, R, Qn
constexpr int RING = 2 * STAGE;
constexpr int EPITCH = 64 + 4;           // floats per staged accumulator row (16-byte aligned, conflict-free)
constexpr int ESTG = 32 * EPITCH * 4;    // bytes per wavefront: one 32-row band
constexpr int SMEM = RING + 4 * ESTG;
constexpr int NPIECE = 8;                // epilogue pieces per tile: 2 outputs x 2 bands x 2 halves
constexpr int PREFETCH = 2;              // pieces whose M / X values are requested ahead

struct FusedArgs {
  const bf16_t* S;        // P:  [batch][tiles_s * 128][r]
  const bf16_t* D1;       // R:  [batch][tiles_d * 128][r]
  const bf16_t* D2;       // Qn: same
  DaPtrTable mtab, xtab;  // per-matrix momentum (bf16) and weights (bf16 or fp32), row pitch ldo; by value: the
                          // lookups are scalar loads from the kernel-argument segment
  long long sS, sD;       // batch strides (elements)
  int tiles_s, tiles_d;
  int r, ldo, total;
  float ef_alpha, decay, neg_lr;
};

struct FTile { int b, ts, td; };

__device__ __forceinline__ FTile decode(const FusedArgs& a, int t) {
  const int per = a.tiles_s * a.tiles_d;
  FTile f;
  f.b = t / per;
  t -= f.b * per;
  if ((a.tiles_s & 7) == 0 && (a.tiles_d & 3) == 0) {
    // 8 x 4 super-tiles: the 32 tiles an XCD works on at a time share 8 P panels and 4 R / Qn panel pairs
    const int sup = t >> 5, within = t & 31;
    const int per_row = a.tiles_d >> 2;
    const int sr = sup / per_row, sc = sup - sr * per_row;
    f.ts = sr * 8 + (within >> 2);
    f.td = sc * 4 + (within & 3);
  } else {
    f.ts = t / a.tiles_d;
    f.td = t - f.ts * a.tiles_d;
  }
  return f;
}

// workgroup barrier that does not wait for outstanding global loads / stores (the prefetched M / X values and the
// epilogue's stores stay in flight); LDS traffic of the wavefront is complete
__device__ __forceinline__ void group_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One stage (64 k) of the three operand tiles of tile `f` into the ring buffer `st`, by the four wavefronts of a
// group: wave-instruction (gw + 4 i) of an operand fills its 1 KB block of 8 rows.
__device__ __forceinline__ void dma_stage(const FusedArgs& a, const FTile& f, int kt, char* st, int gw, int lane) {
  const int row = gw * 8 + (lane >> 3);
  const unsigned doff = (unsigned)(row * a.r + kc_swizzle(lane & 7, row) * 8) * 2u;
  const unsigned dstep = (unsigned)(32 * a.r) * 2u;   // 32 rows further: the swizzle term is unchanged
  const char* bs = reinterpret_cast<const char*>(a.S + (long long)f.b * a.sS + (long long)f.ts * FT * a.r) + kt * (BK * 2);
  const char* b1 = reinterpret_cast<const char*>(a.D1 + (long long)f.b * a.sD + (long long)f.td * FT * a.r) + kt * (BK * 2);
  const char* b2 = reinterpret_cast<const char*>(a.D2 + (long long)f.b * a.sD + (long long)f.td * FT * a.r) + kt * (BK * 2);
  const unsigned l = lds_addr(st) + gw * 1024;
#pragma unroll
  for (int i = 0; i < 4; ++i) dma16(bs, doff + i * dstep, l + i * 4096);
#pragma unroll
  for (int i = 0; i < 4; ++i) dma16(b1, doff + i * dstep, l + OPND + i * 4096);
#pragma unroll
  for (int i = 0; i < 4; ++i) dma16(b2, doff + i * dstep, l + 2 * OPND + i * 4096);
}

// The two 16-row passes of piece (band, half) of one output: M / X values of the wavefront's 64 x 64 sub-tile.
template <bool CF32>
__device__ __forceinline__ void load_piece(u32x4_t (&ev)[2][2], const char* obase, long long ldo, int wm0, int wn0,
                                           int band, int half, int lane) {
  constexpr int CSZ = CF32 ? 4 : 2;
  const int lr = lane >> 3, c8 = (lane & 7) * 8;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int m = wm0 + band * 32 + (half * 2 + q) * 8 + lr;
    const char* p = obase + ((long long)m * ldo + wn0 + c8) * CSZ;
    ev[q][0] = ldg16(p);
    if (CF32) ev[q][1] = ldg16(p + 16);
  }
}

// C = r(r(s0 E) + r(s1 r(acc)))  for the 16 rows x 64 columns of piece (band, half); the band's accumulators go
// through the wavefront's LDS staging area first so that C and E move as 16-byte row segments.
template <bool CF32>
__device__ __forceinline__ void do_piece(const f32x16_t (&acc)[2][2], int band, int half, float* stg, char* obase,
                                         long long ldo, int wm0, int wn0, int lane, float s0, float s1,
                                         const u32x4_t (&ev)[2][2]) {
  constexpr int CSZ = CF32 ? 4 : 2;
  const int lr = lane >> 3, c8 = (lane & 7) * 8;
  if (half == 0) {
    float* row = stg + (lane & 31) * EPITCH + (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq)
        *reinterpret_cast<float4*>(row + j * 32 + vq * 8) =
            make_float4(acc[band][j][vq * 4], acc[band][j][vq * 4 + 1], acc[band][j][vq * 4 + 2], acc[band][j][vq * 4 + 3]);
    wave_sync_lds();
  }
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int rr = (half * 2 + q) * 8 + lr;
    const int m = wm0 + band * 32 + rr;
    const float* sp = stg + rr * EPITCH + c8;
    const float4 a0 = *reinterpret_cast<const float4*>(sp);
    const float4 a1 = *reinterpret_cast<const float4*>(sp + 4);
    float v[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    char* Cp = obase + ((long long)m * ldo + wn0 + c8) * CSZ;
    if (CF32) {
      u32x4_t o[2];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const unsigned w = ev[q][k >> 2][k & 3];
        o[k >> 2][k & 3] = __builtin_bit_cast(unsigned, epi_value<true, true, true>(s0, s1, v[k], __builtin_bit_cast(float, w)));
      }
      stg16(Cp, o[0]);
      stg16(Cp + 16, o[1]);
    } else {
      u32x4_t pk;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const unsigned w = ev[q][0][k];
        pk[k] = epi_pair<true, true, false>(s0, s1, v[2 * k], v[2 * k + 1], w);
      }
      stg16(Cp, pk);
    }
  }
  if (half == 1) wave_sync_lds();
}

// DUAL_A: the matrices are wider than tall (m < n), so M = R P^T: the dual operand (R, Qn) supplies the output
// rows and P the columns.  XF32: fp32 weights.
template <bool DUAL_A, bool XF32>
__global__ __launch_bounds__(512) void dion_ef_update_kernel(FusedArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = wave_uniform(tid >> 6);
  const int grp = wave >> 2, gw = wave & 3;
  const int wm = gw >> 1, wn = gw & 1;
  const int KT = a.r / BK;
  // this workgroup's tiles: first + k * gridDim.x; workgroups are dealt round-robin to the XCDs, so consecutive
  // tiles (which share operand panels) go to workgroups of the same XCD
  const int G = (int)gridDim.x, w = (int)blockIdx.x;
  const int first = (G & 7) == 0 ? (w & 7) * (G >> 3) + (w >> 3) : w;
  const int n_my = first < a.total ? (a.total - first + G - 1) / G : 0;
  float* const stg = reinterpret_cast<float*>(lds + RING) + gw * (32 * EPITCH);
  // operand tiles within a stage: rows of the output come from ra (and rb for the second product), columns from
  // ca (and cb)
  constexpr int R1 = DUAL_A ? OPND : 0, R2 = DUAL_A ? 2 * OPND : 0;
  constexpr int C1 = DUAL_A ? 0 : OPND, C2 = DUAL_A ? 0 : 2 * OPND;

  f32x16_t acc1[2][2], acc2[2][2];     // P R^T and P Qn^T of the wavefront's 64 x 64 sub-tile
  u32x4_t ev[PREFETCH + 1][2][2];      // requested M / X values, ring over the pieces
  FTile mine{0, 0, 0};                 // the tile whose accumulators this group holds,
  char *Mb = nullptr, *Xb = nullptr;   // and the matrices it belongs to

  if (grp == 0 && n_my > 0) {
    dma_stage(a, decode(a, first), 0, lds, gw, lane);
    dma_wait();
  }
  group_barrier();

  for (int s = 0; s <= n_my; ++s) {
    const int ring0 = (s * KT) & 1;    // ring buffer of the slot's first stage
    if ((s & 1) == grp && s < n_my) {
      // ------------------------------------------------------------------ K loop of tile s
      __builtin_amdgcn_s_setprio(2);
      mine = decode(a, first + s * G);
      Mb = static_cast<char*>(a.mtab.p[mine.b]);
      Xb = static_cast<char*>(a.xtab.p[mine.b]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) { acc1[i][j][v] = 0.f; acc2[i][j][v] = 0.f; }
      bf16x8_t fr1[2], fr2[2], fc1[2], fc2[2], gr1[2], gr2[2], gc1[2], gc2[2];
#define DA_FREAD(st, ks, R1v, R2v, C1v, C2v)                                                        \
  do {                                                                                              \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                 \
      R1v[i] = read_frag<FT, false>((st) + R1, wm * 64 + i * 32, (ks), lane);                       \
      if (DUAL_A) R2v[i] = read_frag<FT, false>((st) + R2, wm * 64 + i * 32, (ks), lane);           \
    }                                                                                               \
    _Pragma("unroll") for (int j = 0; j < 2; ++j) {                                                 \
      C1v[j] = read_frag<FT, false>((st) + C1, wn * 64 + j * 32, (ks), lane);                       \
      if (!DUAL_A) C2v[j] = read_frag<FT, false>((st) + C2, wn * 64 + j * 32, (ks), lane);          \
    }                                                                                               \
  } while (0)
#define DA_MMA(R1v, R2v, C1v, C2v)                                                                  \
  do {                                                                                              \
    _Pragma("unroll") for (int i = 0; i < 2; ++i)                                                   \
        _Pragma("unroll") for (int j = 0; j < 2; ++j) {                                             \
      acc1[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(C1v[j], R1v[i], acc1[i][j], 0, 0, 0);    \
      acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(DUAL_A ? C1v[j] : C2v[j],                \
                                                           DUAL_A ? R2v[i] : R1v[i], acc2[i][j], 0, 0, 0); \
    }                                                                                               \
  } while (0)
      DA_FREAD(lds + ring0 * STAGE, 0, fr1, fr2, fc1, fc2);
      for (int kt = 0; kt < KT; ++kt) {
        char* cur = lds + ((ring0 + kt) & 1) * STAGE;
        char* nxt = lds + ((ring0 + kt + 1) & 1) * STAGE;
        const bool more = kt + 1 < KT;
        // the next stage of the ring: of this tile, or the first one of the other group's next tile
        const bool fill = more || s + 1 < n_my;
        if (more) dma_stage(a, mine, kt + 1, nxt, gw, lane);
        else if (fill) dma_stage(a, decode(a, first + (s + 1) * G), 0, nxt, gw, lane);
        DA_FREAD(cur, 1, gr1, gr2, gc1, gc2);
        __builtin_amdgcn_sched_barrier(0);
        DA_MMA(fr1, fr2, fc1, fc2);
        __builtin_amdgcn_sched_barrier(0);
        DA_FREAD(cur, 2, fr1, fr2, fc1, fc2);
        __builtin_amdgcn_sched_barrier(0);
        DA_MMA(gr1, gr2, gc1, gc2);
        __builtin_amdgcn_sched_barrier(0);
        DA_FREAD(cur, 3, gr1, gr2, gc1, gc2);
        __builtin_amdgcn_sched_barrier(0);
        DA_MMA(fr1, fr2, fc1, fc2);
        __builtin_amdgcn_sched_barrier(0);
        if (more) {
          dma_wait();
        } else {
          // the epilogue of this tile starts right after the barrier: request its first M values now (2 loads per
          // piece); loads return in order, so the stage is complete once all but these are back
          const int m0 = (DUAL_A ? mine.td : mine.ts) * FT + wm * 64, n0 = (DUAL_A ? mine.ts : mine.td) * FT + wn * 64;
#pragma unroll
          for (int p = 0; p < PREFETCH; ++p) load_piece<false>(ev[p], Mb, a.ldo, m0, n0, (p >> 1) & 1, p & 1, lane);
          static_assert(PREFETCH == 2, "the wait below counts 2 loads per prefetched piece");
          asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        }
        group_barrier();
        if (more) DA_FREAD(nxt, 0, fr1, fr2, fc1, fc2);
        __builtin_amdgcn_sched_barrier(0);
        DA_MMA(gr1, gr2, gc1, gc2);
        __builtin_amdgcn_sched_barrier(0);
      }
#undef DA_FREAD
#undef DA_MMA
      __builtin_amdgcn_s_setprio(0);
    } else {
      // ------------------------------------------------------------------ epilogue of tile s - 1 (if any)
      const bool have = s >= 1 && ((s - 1) & 1) == grp;
      const int m0 = (DUAL_A ? mine.td : mine.ts) * FT + wm * 64, n0 = (DUAL_A ? mine.ts : mine.td) * FT + wn * 64;
      int bars = 0;
#pragma unroll
      for (int p = 0; p < NPIECE; ++p) {
        if (have) {
          // piece p: output p / 4 (0: momentum, 1: weights), band (p / 2) % 2, half p % 2
          constexpr int slots = PREFETCH + 1;
          const int pn = p + PREFETCH;
          if (pn < NPIECE) {
            if (pn < 4) load_piece<false>(ev[pn % slots], Mb, a.ldo, m0, n0, (pn >> 1) & 1, pn & 1, lane);
            else load_piece<XF32>(ev[pn % slots], Xb, a.ldo, m0, n0, (pn >> 1) & 1, pn & 1, lane);
          }
          if (p < 4) do_piece<false>(acc1, (p >> 1) & 1, p & 1, stg, Mb, a.ldo, m0, n0, lane, 1.f, a.ef_alpha, ev[p % slots]);
          else do_piece<XF32>(acc2, (p >> 1) & 1, p & 1, stg, Xb, a.ldo, m0, n0, lane, a.decay, a.neg_lr, ev[p % slots]);
        }
        const int target = ((p + 1) * KT) / NPIECE;
        for (; bars < target; ++bars) group_barrier();
      }
    }
  }
}

template <bool DUAL_A, bool XF32>
int launch(const FusedArgs& a, hipStream_t s) {
  auto k = dion_ef_update_kernel<DUAL_A, XF32>;
  static DaOncePerDevice configured;
  const int rc_cfg = configured.run([&]() -> int {
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, SMEM));
    return DA_OK;
  });
  if (rc_cfg) return rc_cfg;
  int grid = da_cu_count();
  if (grid > a.total) grid = a.total;
  hipLaunchKernelGGL(k, dim3((unsigned)grid), dim3(512), SMEM, s, a);
  return da_launch_status();
}

}  // namespace

bool da_dion_ef_update_applicable(int mp, int np, int r, int m_dtype) {
  // (offsets within a matrix are 32-bit in the kernel: fp32 weights of mp x np elements must stay below 4 GiB)
  return m_dtype == DA_BF16 && mp % FT == 0 && np % FT == 0 && r % BK == 0 && r >= BK &&
         (long long)mp * np * 4 < (1LL << 32);
}

int da_dion_ef_update(const void* P, const void* R, const void* Qn, const DaPtrTable& tabM, const DaPtrTable& tabX, int batch,
                      int mp, int np, int r, int ldo, int transposed, int x_dtype, float ef_alpha, float decay,
                      float scaled_lr, hipStream_t s) {
  if (!P || !R || !Qn || batch <= 0 || batch > DA_MAX_PTRS) return DA_ERR_ARG;
  if (!da_dion_ef_update_applicable(mp, np, r, DA_BF16)) return DA_ERR_ALIGN;
  if (x_dtype != DA_BF16 && x_dtype != DA_F32) return DA_ERR_DTYPE;
  FusedArgs a{};
  a.S = static_cast<const bf16_t*>(P);
  a.D1 = static_cast<const bf16_t*>(R);
  a.D2 = static_cast<const bf16_t*>(Qn);
  a.mtab = tabM; a.xtab = tabX;
  a.sS = (long long)mp * r; a.sD = (long long)np * r;
  a.tiles_s = mp / FT; a.tiles_d = np / FT;
  a.r = r; a.ldo = ldo;
  const long long total = (long long)a.tiles_s * a.tiles_d * batch;
  if (total > 0x7fffffffLL) return DA_ERR_LIMIT;
  a.total = (int)total;
  a.ef_alpha = ef_alpha; a.decay = decay; a.neg_lr = -scaled_lr;
  const bool xf = x_dtype == DA_F32;
  if (transposed) return xf ? launch<true, true>(a, s) : launch<true, false>(a, s);
  return xf ? launch<false, true>(a, s) : launch<false, false>(a, s);
}
