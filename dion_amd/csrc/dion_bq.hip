// B = M + G and P = B Q in one launch (reference dion/dion.py:794 `torch._foreach_add_(M, G)` and 801
// `P = M_batch @ Q_batch`, bf16 momentum and gradients).
//
// Done as two launches, the step reads M and G and writes B (= the new M) in one pass and reads B again for the
// product.  Here the product's row operand is formed on the way into LDS -- every 16-byte chunk of M and of G is
// loaded once, added with the reference's one rounding, stored into the operand stage and back over M -- so the
// addition's three passes over the matrix run under the product's matrix-core work and B is not read again.
//
// A workgroup owns 256 rows of B (all of K) and computes the first 256 columns of P with the summing K loop, which
// writes B back; no other workgroup touches those rows, so no element of M is added to twice.  Columns of P beyond
// the first 256 (ranks above 256) are a plain product on the finished B, launched by the caller behind this one.
// The tile code is the batched kernel's, with the same order of summation: P has the same bits as from the two
// launches.
#include "dion.h"
#include "gemm_bf16_tile.h"

namespace {

typedef Cfg<256, 2, 4> Big;

struct BqArgs {
  DaPtrTable m, g;           // momentum (read and written) and gradient of every matrix
  const bf16_t* Q;           // [batch][np][ldq]
  bf16_t* P;                 // [batch][mp][ldq]
  long long sQ, sP;          // elements between consecutive matrices
  int* nonzero;              // [batch]: set to 1 by every workgroup that saw a sum that is not zero
  int mp, np, r, ldq, ldm;   // P = B Q: B is mp x np (row pitch ldm, or np x mp stored rows when transposed), Q np x r
  int faithful;
};

template <bool A_KS>
__global__ __launch_bounds__(Big::NT) void dion_bq_sum_kernel(BqArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int BT = Big::BT;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = wave_uniform(tid >> 6);
  const int wm = wave / Big::WGN, wn = wave % Big::WGN;
  const int row_blocks = a.mp / BT;
  const int b = (int)blockIdx.x / row_blocks;
  const int ti = (int)blockIdx.x - b * row_blocks;
  const int m0 = ti * BT;
  bf16_t* M = static_cast<bf16_t*>(a.m.p[b]);
  const bf16_t* G = static_cast<const bf16_t*>(a.g.p[b]);
  const bf16_t* Q = a.Q + (long long)b * a.sQ;

  GemmDesc d{};
  d.batch = 1; d.c_dtype = DA_BF16; d.faithful = a.faithful;
  d.M = a.mp; d.N = a.r; d.K = a.np;
  d.lda = a.ldm; d.ldb = a.ldq; d.ldc = a.ldq;
  d.a_kstrided = A_KS ? 1 : 0; d.b_kstrided = 1;
  d.C = a.P + (long long)b * a.sP;
  d.epilogue = DA_EPI_STORE; d.s0 = 0.f; d.s1 = 1.f;

  bool any = false;
  Big::acc_t acc[Big::TMI][Big::TNJ];
  gemm_tile_k_loop_sum<Big, A_KS>(acc, d, M, G, Q, d.K, m0, 0, lds, tid, lane, wave, wm, wn, true, any);
  epilogue<Big, false, false>(acc, d, lds, 0, ti, 0, m0, 0, wave, lane, wm, wn);
  // every writer stores the same value: no atomic needed
  if (__any(any) && lane == 0) a.nonzero[b] = 1;
}

// Bytes from the first to the last element a workgroup reads of one operand (256 rows, all of K): the direct-to-LDS
// loads address them with 32-bit offsets.
long long span_bytes(bool kstrided, long long ld, long long K) {
  return 2 * (kstrided ? (K - 1) * ld + 256 : 255 * ld + K);
}

}  // namespace

// bf16 momentum and gradients; whole 256-row tiles of B; K in whole stages; the rank a multiple of 8 (the working
// matrices' pitch).  Ranks above 256 leave the other column tiles to a second launch: worth it only while the row
// blocks alone keep most of the compute units busy.
bool da_dion_bq_sum_applicable(int batch, int mp, int np, int r, int ldm, int transposed, int m_dtype, int g_dtype) {
  if (m_dtype != DA_BF16 || g_dtype != DA_BF16) return false;
  if (mp % 256 || np % BK || (r & 7) || r < 8) return false;
  if (span_bytes(true, r, np) >= (1LL << 32) || span_bytes(transposed != 0, ldm, np) >= (1LL << 32)) return false;
  if (2LL * mp * np >= (1LL << 32)) return false;   // (the summing loop addresses a matrix with 32-bit byte offsets)
  const int col_tiles = (r + 255) / 256;
  const long long groups = (long long)batch * (mp / 256);
  if (groups > 0x7fffffffLL) return false;
  return col_tiles == 1 || groups * 5 >= 4LL * da_cu_count();
}

int da_dion_bq_sum(const DaPtrTable& tabM, const DaPtrTable& tabG, const void* Q, void* P, long long sQ, long long sP,
                   int* nonzero, int batch, int mp, int np, int r, int ldq, int ldm, int transposed, int faithful,
                   hipStream_t s) {
  if (batch < 1 || batch > DA_MAX_PTRS) return DA_ERR_LIMIT;
  if (!da_dion_bq_sum_applicable(batch, mp, np, r, ldm, transposed, DA_BF16, DA_BF16) || (ldq & 7) || (ldm & 7) || ldq != r)
    return DA_ERR_ARG;
  constexpr int stage2 = 2 * (Tile<256, false>::bytes + Tile<256, true>::bytes);
  constexpr int epi = (Big::NT / 64) * 32 * (Big::WCOLS + 4) * 4;
  constexpr int smem = stage2 > epi ? stage2 : epi;
  static DaOncePerDevice configured;
  const int rc = configured.run([&]() -> int {
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(dion_bq_sum_kernel<false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(dion_bq_sum_kernel<true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return DA_OK;
  });
  if (rc) return rc;
  BqArgs a{};
  a.m = tabM; a.g = tabG;
  a.Q = static_cast<const bf16_t*>(Q); a.P = static_cast<bf16_t*>(P);
  a.sQ = sQ; a.sP = sP; a.nonzero = nonzero;
  a.mp = mp; a.np = np; a.r = r; a.ldq = ldq; a.ldm = ldm; a.faithful = faithful;
  const unsigned grid = (unsigned)((long long)batch * (mp / 256));
  if (transposed) hipLaunchKernelGGL(dion_bq_sum_kernel<true>, dim3(grid), dim3(Big::NT), smem, s, a);
  else hipLaunchKernelGGL(dion_bq_sum_kernel<false>, dim3(grid), dim3(Big::NT), smem, s, a);
  return da_launch_status();
}
