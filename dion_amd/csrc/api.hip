// C ABI entry points (declared in include/dion_amd.h) and the host-side drivers that chain
// the kernels of one Newton-Schulz / Muon bucket on a stream.
#include "../../include/dion_amd.h"
#include "common.h"
#include <cstdlib>
#include <cstring>
#include <mutex>
#include "elementwise.h"
#include "prof.h"
#include "dion.h"
#include "ns_flow.h"

namespace {

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Workspace carve-up for one chunk of `cb` wide matrices (mw x nw).
// Row pitch of a working matrix with n columns.  A pitch that is a multiple of 4 KiB puts every row
// of an operand tile on the same L2 channel (measured: 4096-wide bf16 operands run 17 % slower than
// with 128 bytes of padding), so such rows get 128 bytes more.
inline int padded_pitch(int n, size_t esz) { return ((size_t)n * esz) % 4096 == 0 ? n + (int)(128 / esz) : n; }

struct NsLayout {
  int mw = 0, nw = 0, tiles = 0;
  int ldx = 0, lda = 0;   // row pitches of the mw x nw iterates and of the mw x mw Gram / polynomial
  size_t esz = 0;
  size_t x_bytes = 0, a_bytes = 0, part_bytes = 0, flow_bytes = 0;  // per matrix
  size_t per_matrix = 0;
  NsLayout() {}
  NsLayout(int m, int n, int dtype) {
    mw = m < n ? m : n;
    nw = m < n ? n : m;
    tiles = da_stage_tiles(m, n);
    esz = dtype == DA_BF16 ? 2 : 4;
    // no padding between matrices: with every pitch a multiple of 8 each one starts 16-byte aligned
    ldx = padded_pitch(nw, esz);
    lda = padded_pitch(mw, esz);
    x_bytes = (size_t)mw * ldx * esz;
    a_bytes = (size_t)mw * lda * esz;
    part_bytes = align_up((size_t)tiles * sizeof(float) + sizeof(float), 256);
    // control words of the persistent Newton-Schulz kernel: cb * flow_bytes >= da_ns_flow_ctl_bytes(cb) for cb >= 1
    // (+ 16: one slot of the table of weight pointers that the last product's epilogue updates)
    flow_bytes = DA_FLOW_CTR_STRIDE * sizeof(int) + 256 + 16;
    per_matrix = 2 * x_bytes + 2 * a_bytes + part_bytes + flow_bytes;
  }
  int chunk(int batch, size_t ws_bytes) const {
    size_t c = ws_bytes / per_matrix;
    if (c > (size_t)batch) c = batch;
    if (c > DA_MAX_PTRS) c = DA_MAX_PTRS;
    return (int)c;
  }
  size_t recommended(int batch) const {
    size_t c = ((size_t)4 << 30) / per_matrix;
    if (c < 1) c = 1;
    if (c > (size_t)batch) c = batch;
    if (c > DA_MAX_PTRS) c = DA_MAX_PTRS;
    return c * per_matrix;
  }
};

struct NsBuffers {
  char *x0 = nullptr, *x1 = nullptr, *a = nullptr, *b = nullptr;
  float *partials = nullptr, *divisor = nullptr;
  int* flow = nullptr;
  void** xtab = nullptr;   // per-matrix weight pointers (Muon: the last product updates the weights itself)
  NsBuffers() {}
  NsBuffers(const NsLayout& L, void* ws, int cb) {
    char* p = static_cast<char*>(ws);
    x0 = p; p += L.x_bytes * cb;
    x1 = p; p += L.x_bytes * cb;
    a = p; p += L.a_bytes * cb;
    b = p; p += L.a_bytes * cb;
    partials = reinterpret_cast<float*>(p); p += L.part_bytes * cb;
    divisor = partials + (size_t)L.tiles * cb;
    flow = reinterpret_cast<int*>(p);
    xtab = reinterpret_cast<void**>(p + (DA_FLOW_CTR_STRIDE * sizeof(int) + 256) * (size_t)cb);
  }
};

// Executed multiply-adds of one launch (symmetric outputs: upper triangle incl. diagonal).
double gemm_flops(const GemmDesc& d) {
  const double mn = d.symmetric ? 0.5 * (double)d.M * ((double)d.M + 1.0) : (double)d.M * d.N;
  return 2.0 * mn * d.K * d.batch;
}

int gemm_any(const GemmDesc& d, int dtype, hipStream_t s, int kind = DA_PROF_GEMM) {
  DaProfScope prof(kind, gemm_flops(d), s);
  return dtype == DA_BF16 ? da_gemm_bf16(d, s) : da_gemm_f32(d, s);
}

// `n` products of the same form: one grouped launch in bf16, one launch each in fp32.
int gemm_group(const GemmDesc* d, int n, int dtype, hipStream_t s, int kind) {
  double flops = 0.0;
  for (int i = 0; i < n; ++i) flops += gemm_flops(d[i]);
  static const bool nogroup = getenv("DION_AMD_NO_GROUP") != nullptr;
  if (dtype == DA_BF16 && !nogroup) {
    DaProfScope prof(kind, flops, s);
    return da_gemm_bf16_grouped(d, n, s);
  }
  for (int i = 0; i < n; ++i) {
    const int rc = gemm_any(d[i], dtype, s, kind);
    if (rc) return rc;
  }
  return DA_OK;
}

// One set of wide matrices iterated together with others: `cb` matrices of layout L in buffers W.
struct NsSet {
  NsLayout L;
  NsBuffers W;
  int cb = 0;
  // Muon: the last X' = aX + BX does not store its result but applies it to the weights W.xtab[b] (x_dtype, rows x
  // cols as the optimizer holds them: transposed with respect to the wide working matrix when tall)
  int update = 0, x_dtype = 0, tall = 0, x_ld = 0;
  float decay = 1.f, step = 1.f;
};

// steps x { A = X X^T ; B = b A + c A A ; X' = a X + B X } on up to DA_MAX_GROUPS sets of wide
// matrices at once (each of the three products is one grouped launch over all sets).
// Returns in result[i] which of x0 / x1 of set i holds the final iterate, and in *poison (if asked for) a device word
// that is non-zero when the iterates are invalid (null: there is no such word).  With `updated` given and every set
// carrying its weight table, the last product applies the weight update itself where its launch allows that
// (*updated = true: result[] then holds nothing of use and the caller skips its own update pass).
int ns_iterate(const NsSet* sets, int nsets, int dtype, const float* coeffs, int steps, int faithful, hipStream_t s,
               char** result, const int** poison = nullptr, bool* updated = nullptr) {
  if (nsets < 1 || nsets > DA_MAX_GROUPS) return DA_ERR_ARG;
  if (poison) *poison = nullptr;
  if (updated) *updated = false;
  bool want_update = updated != nullptr && dtype == DA_BF16 && steps >= 1;
  for (int i = 0; i < nsets; ++i) want_update = want_update && sets[i].update;
  if (dtype == DA_BF16 && steps >= 1) {
    // many small matrices: all iterations of all sets as one persistent launch (ns_flow.hip); the sets are dealt to
    // its queues most expensive first
    DaNsFlowGroup fg[DA_MAX_GROUPS];
    int order[DA_MAX_GROUPS];
    for (int i = 0; i < nsets; ++i) order[i] = i;
    auto cost = [&](int i) { const NsLayout& L = sets[i].L; return (double)L.mw * L.mw * (3.0 * L.nw + L.mw); };
    for (int i = 1; i < nsets; ++i)
      for (int j = i; j > 0 && cost(order[j - 1]) < cost(order[j]); --j) { const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
    for (int k = 0; k < nsets; ++k) {
      const NsLayout& L = sets[order[k]].L;
      const NsBuffers& W = sets[order[k]].W;
      const NsSet& S = sets[order[k]];
      fg[k] = DaNsFlowGroup{W.x0, W.x1, W.a, W.b, (long long)(L.x_bytes / L.esz), (long long)(L.a_bytes / L.esz),
                            L.mw, L.nw, L.ldx, L.lda, S.cb, W.flow,
                            want_update ? W.xtab : nullptr, S.x_dtype, S.x_ld, S.tall, S.decay, S.step};
    }
    // (the persistent kernel updates bf16 weights only: others get the separate pass)
    bool flow_update = want_update;
    for (int i = 0; i < nsets; ++i) flow_update = flow_update && sets[i].x_dtype == DA_BF16;
    if (!flow_update)
      for (int k = 0; k < nsets; ++k) fg[k].upd_tab = nullptr;
    if (da_ns_flow_applicable(fg, nsets, steps, faithful)) {
      double flops = 0.0;
      for (int i = 0; i < nsets; ++i) {
        const NsLayout& L = sets[i].L;
        flops += (double)steps * sets[i].cb * ((double)L.mw * (L.mw + 1.0) * (L.nw + L.mw) + 2.0 * L.mw * L.mw * L.nw);
      }
      DaProfScope prof(DA_PROF_NS_FLOW, flops, s);
      const int rc = da_ns_flow(fg, nsets, coeffs, steps, faithful, s);
      if (rc) return rc;
      for (int i = 0; i < nsets; ++i) result[i] = (steps & 1) ? sets[i].W.x1 : sets[i].W.x0;
      if (poison) *poison = da_ns_flow_status_word(fg);
      if (flow_update) *updated = true;
      return DA_OK;
    }
  }
  char *x[DA_MAX_GROUPS], *y[DA_MAX_GROUPS];
  for (int i = 0; i < nsets; ++i) { x[i] = sets[i].W.x0; y[i] = sets[i].W.x1; }
  for (int it = 0; it < steps; ++it) {
    const float a = coeffs[3 * it], b = coeffs[3 * it + 1], c = coeffs[3 * it + 2];
    GemmDesc g[DA_MAX_GROUPS];
    // A = X X^T   (symmetric output, k = nw)
    for (int i = 0; i < nsets; ++i) {
      const NsLayout& L = sets[i].L;
      const NsBuffers& W = sets[i].W;
      const long long sx = (long long)(L.x_bytes / L.esz), sa = (long long)(L.a_bytes / L.esz);
      g[i] = GemmDesc{};
      g[i].batch = sets[i].cb; g[i].c_dtype = dtype; g[i].faithful = faithful;
      g[i].A = x[i]; g[i].B = x[i]; g[i].C = W.a; g[i].E = nullptr;
      g[i].sA = sx; g[i].sB = sx; g[i].sC = sa; g[i].sE = 0;
      g[i].lda = L.ldx; g[i].ldb = L.ldx; g[i].ldc = L.lda; g[i].lde = 0;
      g[i].M = L.mw; g[i].N = L.mw; g[i].K = L.nw;
      g[i].a_kstrided = 0; g[i].b_kstrided = 0; g[i].symmetric = 1;
      g[i].epilogue = DA_EPI_STORE; g[i].s0 = 0.f; g[i].s1 = 1.f;
    }
    int rc = gemm_group(g, nsets, dtype, s, DA_PROF_NS_SYRK);
    if (rc) return rc;
    // B = b A + c A A^T   (A symmetric, so A A = A A^T: both operands k-contiguous)
    for (int i = 0; i < nsets; ++i) {
      const NsLayout& L = sets[i].L;
      const NsBuffers& W = sets[i].W;
      const long long sa = (long long)(L.a_bytes / L.esz);
      g[i].A = W.a; g[i].B = W.a; g[i].C = W.b; g[i].E = W.a;
      g[i].sA = sa; g[i].sB = sa; g[i].sC = sa; g[i].sE = sa;
      g[i].lda = L.lda; g[i].ldb = L.lda; g[i].ldc = L.lda; g[i].lde = L.lda;
      g[i].M = L.mw; g[i].N = L.mw; g[i].K = L.mw;
      g[i].epilogue = DA_EPI_AXPBY; g[i].s0 = b; g[i].s1 = c;
    }
    rc = gemm_group(g, nsets, dtype, s, DA_PROF_NS_POLY);
    if (rc) return rc;
    // X' = a X + B X   (B symmetric: k-contiguous; X is the k-strided operand)
    for (int i = 0; i < nsets; ++i) {
      const NsLayout& L = sets[i].L;
      const NsBuffers& W = sets[i].W;
      const long long sx = (long long)(L.x_bytes / L.esz), sa = (long long)(L.a_bytes / L.esz);
      g[i].A = W.b; g[i].B = x[i]; g[i].C = y[i]; g[i].E = x[i];
      g[i].sA = sa; g[i].sB = sx; g[i].sC = sx; g[i].sE = sx;
      g[i].lda = L.lda; g[i].ldb = L.ldx; g[i].ldc = L.ldx; g[i].lde = L.ldx;
      g[i].M = L.mw; g[i].N = L.nw; g[i].K = L.mw;
      g[i].a_kstrided = 0; g[i].b_kstrided = 1; g[i].symmetric = 0;
      g[i].epilogue = DA_EPI_AXPBY; g[i].s0 = a; g[i].s1 = 1.f;
    }
    if (want_update && it + 1 == steps && da_gemm_bf16_all_interior(g, nsets)) {
      for (int i = 0; i < nsets; ++i) {
        g[i].upd_tab = sets[i].W.xtab; g[i].upd_dtype = sets[i].x_dtype; g[i].upd_ld = sets[i].x_ld;
        g[i].upd_transposed = sets[i].tall; g[i].upd_decay = sets[i].decay; g[i].upd_step = sets[i].step;
      }
      *updated = true;
    }
    rc = gemm_group(g, nsets, dtype, s, DA_PROF_NS_AXPY);
    if (rc) return rc;
    for (int i = 0; i < nsets; ++i) { char* t = x[i]; x[i] = y[i]; y[i] = t; }
  }
  for (int i = 0; i < nsets; ++i) result[i] = x[i];
  return DA_OK;
}

int ns_iterate(const NsLayout& L, const NsBuffers& W, int cb, int dtype, const float* coeffs, int steps,
               int faithful, hipStream_t s, char** result, const int** poison = nullptr) {
  NsSet one;
  one.L = L; one.W = W; one.cb = cb;
  return ns_iterate(&one, 1, dtype, coeffs, steps, faithful, s, result, poison);
}

// The weights of `c` matrices starting at X[0] as a device table at `dst`, and the set's update parameters.
int ns_set_update(NsSet& set, void* const* X, int first, int c, int m, int n, int x_dtype, float decay, float step,
                  hipStream_t s) {
  DaPtrTable t{};
  for (int j = 0; j < c; ++j) t.p[j] = X[j];
  set.update = 1; set.x_dtype = x_dtype; set.tall = m > n ? 1 : 0; set.x_ld = n; set.decay = decay; set.step = step;
  return da_upload_ptrs(t, set.W.xtab + first, c, s);
}

// After a persistent launch that updated the weights itself: NaN in all of them if the launch gave up.
int ns_poison_weights(void* const* X, int batch, int m, int n, int x_dtype, const int* poison, hipStream_t s) {
  for (int j0 = 0; j0 < batch; j0 += DA_MAX_PTRS) {
    const int c = batch - j0 < DA_MAX_PTRS ? batch - j0 : DA_MAX_PTRS;
    DaPtrTable t{};
    for (int j = 0; j < c; ++j) t.p[j] = X[j0 + j];
    const int rc = da_poison_if(t, c, (long long)m * n, x_dtype, poison, s);
    if (rc) return rc;
  }
  return DA_OK;
}

int ns_normalize_chunk(const NsLayout& L, const NsBuffers& W, int cb, int dtype, float eps, hipStream_t s) {
  DaProfScope prof(DA_PROF_NORMALIZE, 2.0 * (double)L.mw * L.nw * L.esz * cb, s);  // algorithmic bytes (pad excluded)
  // (the divisor is formed inside the launch from the partial sums: no separate finishing launch)
  return da_normalize_from_partials(W.x0, dtype, (long long)(L.x_bytes / L.esz), cb, nullptr, W.partials, L.tiles, eps, s);
}

bool dtype_ok(int d) { return d == DA_BF16 || d == DA_F32; }

// Run-time options (dion_amd_set_option).  -1: not set by the caller, the environment decides.
std::atomic<int> g_opt_fused_update{-1};

// Error feedback and weight update as one pass (the default) or as two AXPBY products.
bool fused_update_enabled() {
  const int v = g_opt_fused_update.load(std::memory_order_relaxed);
  if (v >= 0) return v != 0;
  static const bool env_off = getenv("DION_AMD_NO_FUSED") != nullptr;
  return !env_off;
}

// B = M + G inside the launch of P = B Q (the default where it applies) or as a pass of its own.
std::atomic<int> g_opt_fused_bq{-1};
bool fused_bq_enabled() {
  const int v = g_opt_fused_bq.load(std::memory_order_relaxed);
  if (v >= 0) return v != 0;
  static const bool env_off = getenv("DION_AMD_NO_FUSED_BQ") != nullptr;
  return !env_off;
}

// Number of slices (1, 2 or 4) of the inner dimension `mp` for the product R = B^T P (np x r per matrix, `cb`
// matrices), by the bf16 launcher's own estimate: workgroup rounds x 64-deep stages per tile, a 256 x 256 tile
// costing 4 per stage on a whole CU and a 128 x 128 tile 3 on half a CU; a sliced product also pays for writing
// and adding its fp32 partial sums.
int btp_slices(int np, int r, int mp, int cb) {
  int best = 1;
  double best_cost = 0.0;
  for (int s = 1; s <= DA_MAX_GROUPS; s *= 2) {
    if (s > 1 && (mp / s < 512 || mp % (s * 64) != 0)) break;
    const long long t256 = (long long)((np + 255) / 256) * ((r + 255) / 256) * cb * s;
    const long long t128 = (long long)((np + 127) / 128) * ((r + 127) / 128) * cb * s;
    const double stages = (double)(mp / s) / 64.0;
    const double big = np >= 256 && r >= 256 ? (double)((t256 + 255) / 256) * stages * 4.0 : 1e30;
    const double small = (double)((t128 + 511) / 512) * stages * 3.0;
    double cost = big < small ? big : small;
    if (s > 1) cost += 32.0 + 8.0 * s;
    if (s == 1 || cost < best_cost) { best = s; best_cost = cost; }
  }
  return best;
}

}  // namespace

extern "C" {

const char* dion_amd_version(void) { return "dion_amd 0.1 (gfx950)"; }

size_t dion_amd_ns_workspace_bytes(int batch, int m, int n, int compute_dtype) {
  if (batch <= 0 || m <= 0 || n <= 0 || !dtype_ok(compute_dtype)) return 0;
  return NsLayout(m, n, compute_dtype).recommended(batch);
}

}  // extern "C"

namespace {

int ns_run(const void* G, int g_dtype, long long g_stride, int ldg, void* out, long long out_stride, int ldo,
           int batch, int m, int n, const float* coeffs, int steps, float eps, int compute_dtype, int faithful,
           void* workspace, size_t workspace_bytes, void* stream) {
  if (!G || !out || !coeffs || !workspace || batch <= 0 || m <= 0 || n <= 0 || steps < 0) return DA_ERR_ARG;
  if (!dtype_ok(g_dtype) || !dtype_ok(compute_dtype)) return DA_ERR_DTYPE;
  if ((m | n | ldg | ldo) & 7) return DA_ERR_ALIGN;
  if ((g_stride | out_stride) & 7) return DA_ERR_ALIGN;
  // matrices move as 16-byte chunks; only the workspace, which the library carves up itself, needs 256
  if (((uintptr_t)G | (uintptr_t)out) & 15) return DA_ERR_ALIGN;
  if ((uintptr_t)workspace & 255) return DA_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const NsLayout L(m, n, compute_dtype);
  const int chunk = L.chunk(batch, workspace_bytes);
  if (chunk < 1) return DA_ERR_WORKSPACE;
  const size_t gsz = g_dtype == DA_BF16 ? 2 : 4;
  for (int b0 = 0; b0 < batch; b0 += chunk) {
    const int cb = batch - b0 < chunk ? batch - b0 : chunk;
    const NsBuffers W(L, workspace, cb);
    DaStage st{};
    for (int i = 0; i < cb; ++i)
      st.g.p[i] = const_cast<char*>(static_cast<const char*>(G)) + (size_t)(b0 + i) * g_stride * gsz;
    st.wide = W.x0; st.partials = W.partials;
    st.batch = cb; st.rows = m; st.cols = n; st.ld = ldg; st.ldw = L.ldx;
    st.g_dtype = g_dtype; st.m_dtype = g_dtype; st.w_dtype = compute_dtype;
    st.mu = 0.f; st.nesterov = 0; st.muon = 0;
    int rc;
    {
      DaProfScope prof(DA_PROF_STAGE, (double)m * n * (gsz + L.esz) * cb, s);
      rc = da_stage_wide(st, s);
    }
    if (rc) return rc;
    rc = ns_normalize_chunk(L, W, cb, compute_dtype, eps, s);
    if (rc) return rc;
    char* res = nullptr;
    const int* poison = nullptr;
    rc = ns_iterate(L, W, cb, compute_dtype, coeffs, steps, faithful, s, &res, &poison);
    if (rc) return rc;
    DaUnstage us{};
    us.poison = poison;
    for (int i = 0; i < cb; ++i) us.x.p[i] = static_cast<char*>(out) + (size_t)(b0 + i) * out_stride * L.esz;
    us.wide = res; us.batch = cb; us.rows = m; us.cols = n; us.ld = ldo; us.ldw = L.ldx;
    us.x_dtype = compute_dtype; us.w_dtype = compute_dtype;
    us.decay = 1.f; us.step = 1.f; us.muon = 0;
    {
      DaProfScope prof(DA_PROF_UNSTAGE, 2.0 * (double)m * n * L.esz * cb, s);
      rc = da_unstage(us, s);
    }
    if (rc) return rc;
  }
  return DA_OK;
}

// Working memory of dion_amd_newton_schulz_static: one array per GPU, part of the library's device image (it lives
// as long as the process).  Host code never uses the array's name as an address: `static_scratch()` asks the
// runtime for the device address on the current GPU, once per device, and hands that pointer on.
static __device__ __align__(256) unsigned char scratch[DION_AMD_STATIC_SCRATCH_BYTES];
constexpr int DA_MAX_DEVICES = 64;
void* g_scratch_ptr[DA_MAX_DEVICES];
std::mutex g_scratch_mutex;

int static_scratch(void** ptr) {
  int dev = -1;
  DA_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= DA_MAX_DEVICES) return DA_ERR_LIMIT;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    DA_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return DA_ERR_ARG;
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return DA_OK;
}

}  // namespace

extern "C" {

int dion_amd_newton_schulz(const void* G, int g_dtype, long long g_stride, int ldg, void* out, long long out_stride,
                           int ldo, int batch, int m, int n, const float* coeffs, int steps, float eps,
                           int compute_dtype, int faithful, void* workspace, size_t workspace_bytes, void* stream) {
  return ns_run(G, g_dtype, g_stride, ldg, out, out_stride, ldo, batch, m, n, coeffs, steps, eps, compute_dtype,
                faithful, workspace, workspace_bytes, stream);
}

size_t dion_amd_static_scratch_bytes(void) { return DION_AMD_STATIC_SCRATCH_BYTES; }

int dion_amd_newton_schulz_static(const void* G, int g_dtype, long long g_stride, int ldg, void* out,
                                  long long out_stride, int ldo, int batch, int m, int n, const float* coeffs,
                                  int steps, float eps, int compute_dtype, int faithful, void* stream) {
  if (batch <= 0 || m <= 0 || n <= 0) return DA_ERR_ARG;
  if (!dtype_ok(compute_dtype)) return DA_ERR_DTYPE;
  // one matrix's working set must fit the array (a batch then goes through it in chunks)
  if (NsLayout(m, n, compute_dtype).per_matrix > (size_t)DION_AMD_STATIC_SCRATCH_BYTES) return DA_ERR_LIMIT;
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc) return rc;
  return ns_run(G, g_dtype, g_stride, ldg, out, out_stride, ldo, batch, m, n, coeffs, steps, eps, compute_dtype,
                faithful, ws, DION_AMD_STATIC_SCRATCH_BYTES, stream);
}

int dion_amd_syrk(const void* A, long long a_stride, int lda, void* C, long long c_stride, int ldc, int batch, int m,
                  int k, int dtype, void* stream) {
  if (!dtype_ok(dtype)) return DA_ERR_DTYPE;
  GemmDesc g{};
  g.A = A; g.B = A; g.C = C; g.E = nullptr;
  g.sA = a_stride; g.sB = a_stride; g.sC = c_stride;
  g.lda = lda; g.ldb = lda; g.ldc = ldc;
  g.M = m; g.N = m; g.K = k; g.batch = batch;
  g.symmetric = 1; g.epilogue = DA_EPI_STORE; g.s1 = 1.f; g.faithful = 0; g.c_dtype = dtype;
  return gemm_any(g, dtype, static_cast<hipStream_t>(stream));
}

int dion_amd_sym_poly(const void* A, long long a_stride, int lda, void* C, long long c_stride, int ldc, int batch,
                      int m, float alpha, float beta, int dtype, int faithful, void* stream) {
  if (!dtype_ok(dtype)) return DA_ERR_DTYPE;
  if (A == C) return DA_ERR_ARG;  // mirrored stores would race with operand loads
  GemmDesc g{};
  g.A = A; g.B = A; g.C = C; g.E = A;
  g.sA = a_stride; g.sB = a_stride; g.sC = c_stride; g.sE = a_stride;
  g.lda = lda; g.ldb = lda; g.ldc = ldc; g.lde = lda;
  g.M = m; g.N = m; g.K = m; g.batch = batch;
  g.symmetric = 1; g.epilogue = DA_EPI_AXPBY; g.s0 = beta; g.s1 = alpha; g.faithful = faithful; g.c_dtype = dtype;
  return gemm_any(g, dtype, static_cast<hipStream_t>(stream));
}

int dion_amd_gemm(const void* A, long long a_stride, int lda, int a_kstrided, const void* B, long long b_stride,
                  int ldb, int b_kstrided, void* C, long long c_stride, int ldc, const void* E, long long e_stride,
                  int lde, int batch, int M, int N, int K, int in_dtype, int c_dtype, int epilogue, float s0,
                  float s1, int faithful, void* stream) {
  if (!dtype_ok(in_dtype) || !dtype_ok(c_dtype)) return DA_ERR_DTYPE;
  if (epilogue != DA_EPI_STORE && epilogue != DA_EPI_AXPBY) return DA_ERR_ARG;
  GemmDesc g{};
  g.A = A; g.B = B; g.C = C; g.E = epilogue == DA_EPI_AXPBY ? E : nullptr;
  g.sA = a_stride; g.sB = b_stride; g.sC = c_stride; g.sE = e_stride;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.lde = lde;
  g.M = M; g.N = N; g.K = K; g.batch = batch;
  g.a_kstrided = a_kstrided != 0; g.b_kstrided = b_kstrided != 0; g.symmetric = 0;
  g.epilogue = epilogue; g.s0 = s0; g.s1 = s1; g.faithful = faithful; g.c_dtype = c_dtype;
  return gemm_any(g, in_dtype, static_cast<hipStream_t>(stream));
}

int dion_amd_set_option(const char* name, int value) {
  if (!name) return DA_ERR_ARG;
  if (strcmp(name, "fused_update") == 0) {
    g_opt_fused_update.store(value < 0 ? -1 : (value != 0), std::memory_order_relaxed);
    return DA_OK;
  }
  if (strcmp(name, "fused_bq") == 0) {
    g_opt_fused_bq.store(value < 0 ? -1 : (value != 0), std::memory_order_relaxed);
    return DA_OK;
  }
  if (strcmp(name, "ns_flow") == 0) {
    if (value < -1 || value > 2) return DA_ERR_ARG;
    da_ns_flow_set_mode(value);
    return DA_OK;
  }
  if (strcmp(name, "edge_loop") == 0) {
    da_gemm_bf16_set_edge_loop(value);
    return DA_OK;
  }
  if (strcmp(name, "ns_flow_fail") == 0) {
    da_ns_flow_set_fail(value != 0);
    return DA_OK;
  }
  return DA_ERR_ARG;
}

int dion_amd_ns_flow_trace_enable(int on) {
  da_ns_flow_trace_enable(on);
  return DA_OK;
}
int dion_amd_ns_flow_trace_read(void* host_dst, int max_tiles, int* tiles) {
  return da_ns_flow_trace_read(host_dst, max_tiles, tiles);
}

size_t dion_amd_muon_workspace_bytes(int batch, int m, int n) {
  if (batch <= 0 || m <= 0 || n <= 0) return 0;
  return NsLayout(m, n, DA_BF16).recommended(batch);
}

int dion_amd_muon_step(void* const* X, const void* const* G, void* const* M, int batch, int m, int n, int x_dtype,
                       int g_dtype, float mu, int nesterov, float decay, float adjusted_lr, const float* coeffs,
                       int steps, float eps, int faithful, void* workspace, size_t workspace_bytes, void* stream) {
  if (!X || !G || !M || !coeffs || !workspace || batch <= 0 || m <= 0 || n <= 0 || steps < 0) return DA_ERR_ARG;
  if (!dtype_ok(x_dtype) || !dtype_ok(g_dtype)) return DA_ERR_DTYPE;
  if ((m | n) & 7) return DA_ERR_ALIGN;
  if ((uintptr_t)workspace & 255) return DA_ERR_ALIGN;
  for (int i = 0; i < batch; ++i) {
    if (!X[i] || !G[i] || !M[i]) return DA_ERR_ARG;
    if (((uintptr_t)X[i] | (uintptr_t)G[i] | (uintptr_t)M[i]) & 15) return DA_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const NsLayout L(m, n, DA_BF16);
  const int chunk = L.chunk(batch, workspace_bytes);
  if (chunk < 1) return DA_ERR_WORKSPACE;
  for (int b0 = 0; b0 < batch; b0 += chunk) {
    const int cb = batch - b0 < chunk ? batch - b0 : chunk;
    const NsBuffers W(L, workspace, cb);
    DaStage st{};
    for (int i = 0; i < cb; ++i) {
      st.g.p[i] = const_cast<void*>(G[b0 + i]);
      st.mom.p[i] = M[b0 + i];
    }
    st.wide = W.x0; st.partials = W.partials;
    st.batch = cb; st.rows = m; st.cols = n; st.ld = n; st.ldw = L.ldx;
    st.g_dtype = g_dtype; st.m_dtype = x_dtype; st.w_dtype = DA_BF16;
    st.mu = mu; st.nesterov = nesterov; st.muon = 1;
    const double xsz = x_dtype == DA_BF16 ? 2 : 4, gsz = g_dtype == DA_BF16 ? 2 : 4;
    int rc;
    {
      // algorithmic bytes: read G and M, write M and the bf16 working matrix
      DaProfScope prof(DA_PROF_STAGE, (double)m * n * (gsz + 2 * xsz + 2) * cb, s);
      rc = da_stage_wide(st, s);
    }
    if (rc) return rc;
    rc = ns_normalize_chunk(L, W, cb, DA_BF16, eps, s);
    if (rc) return rc;
    char* res = nullptr;
    const int* poison = nullptr;
    bool updated = false;
    NsSet one;
    one.L = L; one.W = W; one.cb = cb;
    rc = ns_set_update(one, X + b0, 0, cb, m, n, x_dtype, decay, adjusted_lr, s);
    if (rc) return rc;
    rc = ns_iterate(&one, 1, DA_BF16, coeffs, steps, faithful, s, &res, &poison, &updated);
    if (rc) return rc;
    if (updated) {
      if (poison) {
        rc = ns_poison_weights(X + b0, cb, m, n, x_dtype, poison, s);
        if (rc) return rc;
      }
      continue;
    }
    DaUnstage us{};
    us.poison = poison;
    for (int i = 0; i < cb; ++i) us.x.p[i] = X[b0 + i];
    us.wide = res; us.batch = cb; us.rows = m; us.cols = n; us.ld = n; us.ldw = L.ldx;
    us.x_dtype = x_dtype; us.w_dtype = DA_BF16;
    us.decay = decay; us.step = adjusted_lr; us.muon = 1;
    {
      // algorithmic bytes: read X and the bf16 result, write X
      DaProfScope prof(DA_PROF_UNSTAGE, (double)m * n * (2 * xsz + 2) * cb, s);
      rc = da_unstage(us, s);
    }
    if (rc) return rc;
  }
  return DA_OK;
}

int dion_amd_muon_pre(const void* const* G, void* const* M, void* const* U, int batch, int m, int n, int g_dtype,
                      int m_dtype, float mu, int nesterov, void* stream) {
  if (!G || !M || !U || batch <= 0 || m <= 0 || n <= 0) return DA_ERR_ARG;
  if (!dtype_ok(g_dtype) || !dtype_ok(m_dtype)) return DA_ERR_DTYPE;
  if (n & 7) return DA_ERR_ALIGN;
  for (int i = 0; i < batch; ++i) {
    if (!G[i] || !M[i] || !U[i]) return DA_ERR_ARG;
    if (((uintptr_t)G[i] | (uintptr_t)M[i] | (uintptr_t)U[i]) & 15) return DA_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const double gsz = g_dtype == DA_BF16 ? 2 : 4, msz = m_dtype == DA_BF16 ? 2 : 4;
  for (int b0 = 0; b0 < batch; b0 += DA_MAX_PTRS) {
    const int cb = batch - b0 < DA_MAX_PTRS ? batch - b0 : DA_MAX_PTRS;
    DaStage st{};
    for (int i = 0; i < cb; ++i) {
      st.g.p[i] = const_cast<void*>(G[b0 + i]);
      st.mom.p[i] = M[b0 + i];
      st.wtab.p[i] = U[b0 + i];
    }
    st.use_wtab = 1; st.wide = nullptr; st.partials = nullptr;
    st.batch = cb; st.rows = m; st.cols = n; st.ld = n; st.ldw = n;
    st.g_dtype = g_dtype; st.m_dtype = m_dtype; st.w_dtype = DA_BF16;
    st.mu = mu; st.nesterov = nesterov; st.muon = 1;
    DaProfScope prof(DA_PROF_STAGE, (double)m * n * (gsz + 2 * msz + 2) * cb, s);
    const int rc = da_stage_wide(st, s);
    if (rc) return rc;
  }
  return DA_OK;
}

int dion_amd_muon_post(void* const* X, const void* const* O, int batch, int m, int n, int x_dtype, int o_dtype,
                       float decay, float adjusted_lr, void* stream) {
  if (!X || !O || batch <= 0 || m <= 0 || n <= 0) return DA_ERR_ARG;
  if (!dtype_ok(x_dtype) || !dtype_ok(o_dtype)) return DA_ERR_DTYPE;
  if (n & 7) return DA_ERR_ALIGN;
  for (int i = 0; i < batch; ++i) {
    if (!X[i] || !O[i]) return DA_ERR_ARG;
    if (((uintptr_t)X[i] | (uintptr_t)O[i]) & 15) return DA_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const double xsz = x_dtype == DA_BF16 ? 2 : 4;
  for (int b0 = 0; b0 < batch; b0 += DA_MAX_PTRS) {
    const int cb = batch - b0 < DA_MAX_PTRS ? batch - b0 : DA_MAX_PTRS;
    DaUnstage us{};
    for (int i = 0; i < cb; ++i) {
      us.x.p[i] = X[b0 + i];
      us.wtab.p[i] = const_cast<void*>(O[b0 + i]);
    }
    us.use_wtab = 1; us.wide = nullptr;
    us.batch = cb; us.rows = m; us.cols = n; us.ld = n; us.ldw = n;
    us.x_dtype = x_dtype; us.w_dtype = o_dtype;
    us.decay = decay; us.step = adjusted_lr; us.muon = 1;
    DaProfScope prof(DA_PROF_UNSTAGE, (double)m * n * (2 * xsz + (o_dtype == DA_BF16 ? 2 : 4)) * cb, s);
    const int rc = da_unstage(us, s);
    if (rc) return rc;
  }
  return DA_OK;
}

int dion_amd_gemm_plan(int M, int N, int K, int lda, int a_kstrided, int ldb, int b_kstrided) {
  if (M <= 0 || N <= 0 || K <= 0 || lda <= 0 || ldb <= 0) return DA_ERR_ARG;
  GemmDesc g{};
  g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.batch = 1;
  g.a_kstrided = a_kstrided != 0; g.b_kstrided = b_kstrided != 0;
  return da_gemm_bf16_plan(g);
}

size_t dion_amd_muon_buckets_workspace_bytes(const dion_amd_muon_bucket* buckets, int nbuckets) {
  if (!buckets || nbuckets <= 0) return 0;
  size_t worst = 0;
  for (int r0 = 0; r0 < nbuckets; r0 += DA_MAX_GROUPS) {
    size_t need = 0;
    for (int i = r0; i < nbuckets && i < r0 + DA_MAX_GROUPS; ++i) {
      if (buckets[i].batch <= 0 || buckets[i].m <= 0 || buckets[i].n <= 0) return 0;
      need += align_up(NsLayout(buckets[i].m, buckets[i].n, DA_BF16).per_matrix * (size_t)buckets[i].batch, 256);
    }
    if (need > worst) worst = need;
  }
  return worst;
}

int dion_amd_muon_step_buckets(const dion_amd_muon_bucket* buckets, int nbuckets, int x_dtype, int g_dtype, float mu,
                               int nesterov, const float* coeffs, int steps, float eps, int faithful,
                               void* workspace, size_t workspace_bytes, void* stream) {
  if (!buckets || nbuckets <= 0 || !coeffs || !workspace || steps < 0) return DA_ERR_ARG;
  if (!dtype_ok(x_dtype) || !dtype_ok(g_dtype)) return DA_ERR_DTYPE;
  if ((uintptr_t)workspace & 255) return DA_ERR_ALIGN;
  for (int i = 0; i < nbuckets; ++i) {
    const dion_amd_muon_bucket& k = buckets[i];
    if (!k.X || !k.G || !k.M || k.batch <= 0 || k.m <= 0 || k.n <= 0) return DA_ERR_ARG;
    if ((k.m | k.n) & 7) return DA_ERR_ALIGN;
    for (int j = 0; j < k.batch; ++j) {
      if (!k.X[j] || !k.G[j] || !k.M[j]) return DA_ERR_ARG;
      if (((uintptr_t)k.X[j] | (uintptr_t)k.G[j] | (uintptr_t)k.M[j]) & 15) return DA_ERR_ALIGN;
    }
  }
  if (workspace_bytes < dion_amd_muon_buckets_workspace_bytes(buckets, nbuckets)) return DA_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const double xsz = x_dtype == DA_BF16 ? 2 : 4, gsz = g_dtype == DA_BF16 ? 2 : 4;
  for (int r0 = 0; r0 < nbuckets; r0 += DA_MAX_GROUPS) {
    const int nr = nbuckets - r0 < DA_MAX_GROUPS ? nbuckets - r0 : DA_MAX_GROUPS;
    // carve the workspace: every bucket of this round keeps all of its matrices resident
    NsSet sets[DA_MAX_GROUPS];
    char* p = static_cast<char*>(workspace);
    for (int i = 0; i < nr; ++i) {
      const dion_amd_muon_bucket& k = buckets[r0 + i];
      const NsLayout L(k.m, k.n, DA_BF16);
      sets[i].L = L;
      sets[i].W = NsBuffers(L, p, k.batch);
      sets[i].cb = k.batch;
      p += align_up(L.per_matrix * (size_t)k.batch, 256);
    }
    // momentum update, bf16 staging in wide orientation, Frobenius partial sums; then normalise
    for (int i = 0; i < nr; ++i) {
      const dion_amd_muon_bucket& k = buckets[r0 + i];
      const NsLayout& L = sets[i].L;
      const NsBuffers& W = sets[i].W;
      for (int j0 = 0; j0 < k.batch; j0 += DA_MAX_PTRS) {
        const int c = k.batch - j0 < DA_MAX_PTRS ? k.batch - j0 : DA_MAX_PTRS;
        DaStage st{};
        for (int j = 0; j < c; ++j) {
          st.g.p[j] = const_cast<void*>(k.G[j0 + j]);
          st.mom.p[j] = k.M[j0 + j];
        }
        st.wide = W.x0 + (size_t)j0 * L.x_bytes;
        st.partials = W.partials + (size_t)j0 * L.tiles;
        st.batch = c; st.rows = k.m; st.cols = k.n; st.ld = k.n; st.ldw = L.ldx;
        st.g_dtype = g_dtype; st.m_dtype = x_dtype; st.w_dtype = DA_BF16;
        st.mu = mu; st.nesterov = nesterov; st.muon = 1;
        DaProfScope prof(DA_PROF_STAGE, (double)k.m * k.n * (gsz + 2 * xsz + 2) * c, s);
        const int rc = da_stage_wide(st, s);
        if (rc) return rc;
      }
      const int rc = ns_normalize_chunk(L, W, k.batch, DA_BF16, eps, s);
      if (rc) return rc;
    }
    char* res[DA_MAX_GROUPS];
    const int* poison = nullptr;
    bool updated = false;
    // the weights' pointer tables for the last product's epilogue: as few launches as the tables need
    DaPtrUploads up{};
    DaPoisonShape shape{};
    shape.f32 = x_dtype == DA_F32;
    auto flush_uploads = [&](int count, bool poisoning) -> int {
      if (count == 0) return DA_OK;
      return poisoning ? da_poison_multi_if(up, count, shape, poison, s) : da_upload_ptrs_multi(up, count, s);
    };
    auto for_all_tables = [&](bool poisoning) -> int {
      int count = 0;
      for (int i = 0; i < nr; ++i) {
        const dion_amd_muon_bucket& k = buckets[r0 + i];
        for (int j0 = 0; j0 < k.batch; j0 += DA_MAX_PTRS) {
          const int c = k.batch - j0 < DA_MAX_PTRS ? k.batch - j0 : DA_MAX_PTRS;
          for (int j = 0; j < c; ++j) up.t[count].p[j] = k.X[j0 + j];
          up.dst[count] = sets[i].W.xtab + j0;
          up.n[count] = c;
          shape.numel[count] = (long long)k.m * k.n;
          if (++count == DA_MAX_UPLOADS) {
            const int rc = flush_uploads(count, poisoning);
            if (rc) return rc;
            count = 0;
          }
        }
      }
      return flush_uploads(count, poisoning);
    };
    for (int i = 0; i < nr; ++i) {
      const dion_amd_muon_bucket& k = buckets[r0 + i];
      NsSet& S = sets[i];
      S.update = 1; S.x_dtype = x_dtype; S.tall = k.m > k.n ? 1 : 0; S.x_ld = k.n; S.decay = k.decay; S.step = k.adjusted_lr;
    }
    int rc = for_all_tables(false);
    if (rc) return rc;
    rc = ns_iterate(sets, nr, DA_BF16, coeffs, steps, faithful, s, res, &poison, &updated);
    if (rc) return rc;
    if (updated && poison) {
      rc = for_all_tables(true);
      if (rc) return rc;
    }
    for (int i = 0; i < nr && !updated; ++i) {
      const dion_amd_muon_bucket& k = buckets[r0 + i];
      const NsLayout& L = sets[i].L;
      for (int j0 = 0; j0 < k.batch; j0 += DA_MAX_PTRS) {
        const int c = k.batch - j0 < DA_MAX_PTRS ? k.batch - j0 : DA_MAX_PTRS;
        DaUnstage us{};
        for (int j = 0; j < c; ++j) us.x.p[j] = k.X[j0 + j];
        us.wide = res[i] + (size_t)j0 * L.x_bytes;
        us.batch = c; us.rows = k.m; us.cols = k.n; us.ld = k.n; us.ldw = L.ldx;
        us.x_dtype = x_dtype; us.w_dtype = DA_BF16;
        us.decay = k.decay; us.step = k.adjusted_lr; us.muon = 1;
        us.poison = poison;
        DaProfScope prof(DA_PROF_UNSTAGE, (double)k.m * k.n * (2 * xsz + 2) * c, s);
        rc = da_unstage(us, s);
        if (rc) return rc;
      }
    }
  }
  return DA_OK;
}


// ---------------------------------------------------------------------------------------
// Dion
// ---------------------------------------------------------------------------------------
}  // extern "C"

namespace {

struct DionLayout {
  // working orientation: B is mp x np with mp >= np; Q is np x r.  r is the rank rounded up to a multiple
  // of 8 (16-byte rows for every working matrix); the extra columns are zero throughout the step.
  int mp, np, r;
  size_t msz;           // bytes per element of the momentum dtype
  size_t qc, p, rb, qn, orth, sketch, part, small;  // per-matrix byte sizes
  size_t per_matrix;
  DionLayout(int m, int n, int rank, int m_dtype, int sketch_k = 0) {
    mp = m < n ? n : m;
    np = m < n ? m : n;
    r = (rank + 7) & ~7;
    msz = m_dtype == DA_BF16 ? 2 : 4;
    qc = (size_t)np * r * msz;   // exact: the orthonormaliser and the GEMMs take these as
    p = (size_t)mp * r * msz;    // contiguous batches (multiples of 128 bytes by the alignment rule)
    rb = qc;
    qn = qc;
    orth = align_up(da_orth_workspace_bytes(1, mp, r), 256);
    // (a sketched orthonormalisation keeps S P per matrix behind the orthonormaliser's own scratch)
    sketch = sketch_k > 0 ? align_up(da_orth_sketch_extra_bytes(1, sketch_k, r), 256) : 0;
    // fp32 partial sums of R = B^T P when its inner dimension is cut into DA_MAX_GROUPS slices (bf16 only)
    part = m_dtype == DA_BF16 ? (size_t)DA_MAX_GROUPS * np * r * sizeof(float) : 0;
    small = 256;  // flags, info, pointer-table slots
    per_matrix = qc + p + rb + qn + orth + sketch + part + small + 256;
  }
  size_t fixed() const { return 4 * DA_MAX_PTRS * sizeof(void*) + 2 * DA_MAX_PTRS * sizeof(int) + 1024; }
  int chunk(int batch, size_t ws_bytes) const {
    if (ws_bytes < fixed()) return 0;
    size_t c = (ws_bytes - fixed()) / per_matrix;
    if (c > (size_t)batch) c = batch;
    if (c > DA_MAX_PTRS) c = DA_MAX_PTRS;
    return (int)c;
  }
  size_t recommended(int batch) const {
    size_t c = ((size_t)6 << 30) / per_matrix;
    if (c < 1) c = 1;
    if (c > (size_t)batch) c = batch;
    if (c > DA_MAX_PTRS) c = DA_MAX_PTRS;
    return c * per_matrix + fixed();
  }
};

}  // namespace

namespace {
int dion_step_impl(void* const* X, const void* const* G, void* const* M, void* const* Q, int batch, int m, int n,
                   int rank, int x_dtype, int g_dtype, int m_dtype, int q_dtype, float ef_alpha, float decay,
                   float scaled_lr, float eps, int faithful, int power_iters, int qr_method, const void* sketch,
                   int sketch_k, int* info, void* workspace, size_t workspace_bytes, void* stream);
}  // namespace

extern "C" {

int dion_amd_dion_bq_fused(int batch, int m, int n, int rank, int m_dtype, int g_dtype) {
  if (batch <= 0 || m <= 0 || n <= 0 || rank <= 0 || rank > m || rank > n || !dtype_ok(m_dtype) || !dtype_ok(g_dtype)) return 0;
  const DionLayout L(m, n, rank, m_dtype);
  const int cb = batch < DA_MAX_PTRS ? batch : DA_MAX_PTRS;
  return fused_bq_enabled() && da_dion_bq_sum_applicable(cb, L.mp, L.np, L.r, n, m < n ? 1 : 0, m_dtype, g_dtype) ? 1 : 0;
}

size_t dion_amd_dion_workspace_bytes(int batch, int m, int n, int r, int m_dtype) {
  if (batch <= 0 || m <= 0 || n <= 0 || r <= 0 || !dtype_ok(m_dtype)) return 0;
  return DionLayout(m, n, r, m_dtype).recommended(batch);
}

size_t dion_amd_orthonormalize_workspace_bytes(int batch, int rows, int r) {
  if (batch <= 0 || rows <= 0 || r <= 0) return 0;
  return da_orth_workspace_bytes(batch, rows, r) + 256 + (size_t)batch * sizeof(int);
}

int dion_amd_orthonormalize(const void* P, void* out, int dtype, int batch, int rows, int r, int passes,
                            int* info, void* workspace, size_t workspace_bytes, void* stream) {
  return dion_amd_orthonormalize_method(P, out, dtype, batch, rows, r, passes, DA_QR_AUTO, info, workspace,
                                        workspace_bytes, stream);
}

int dion_amd_orthonormalize_method(const void* P, void* out, int dtype, int batch, int rows, int r, int passes,
                                   int qr_method, int* info, void* workspace, size_t workspace_bytes, void* stream) {
  if (!P || !out || !workspace || batch <= 0 || rows <= 0 || r <= 0 || passes < 1 || passes > 3) return DA_ERR_ARG;
  if (qr_method < 0 || qr_method > 2) return DA_ERR_ARG;
  if (!dtype_ok(dtype)) return DA_ERR_DTYPE;
  if (r > rows) return DA_ERR_ARG;
  if (workspace_bytes < dion_amd_orthonormalize_workspace_bytes(batch, rows, r)) return DA_ERR_WORKSPACE;
  if ((uintptr_t)workspace & 255) return DA_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int* inf = info;
  if (!inf) inf = reinterpret_cast<int*>(static_cast<char*>(workspace) + align_up(da_orth_workspace_bytes(batch, rows, r), 256));
  int rc = da_fill_int(inf, batch, 0, s);
  if (rc) return rc;
  DaProfScope prof(DA_PROF_DION_ORTH, 0.0, s);
  return da_orthonormalize(P, out, dtype, batch, rows, r, r, passes, qr_method, workspace, inf, s);
}

size_t dion_amd_orthonormalize_sketch_workspace_bytes(int batch, int rows, int r, int k) {
  if (batch <= 0 || rows <= 0 || r <= 0 || k <= 0) return 0;
  return align_up(dion_amd_orthonormalize_workspace_bytes(batch, rows, r), 256) + da_orth_sketch_extra_bytes(batch, k, r);
}

int dion_amd_orthonormalize_sketch(const void* P, const void* S, void* out, int dtype, int batch, int rows, int r, int k,
                                   int* info, void* workspace, size_t workspace_bytes, void* stream) {
  if (!P || !S || !out || !workspace || batch <= 0 || rows <= 0 || r <= 0 || k < r) return DA_ERR_ARG;
  if (!dtype_ok(dtype)) return DA_ERR_DTYPE;
  if (r > rows) return DA_ERR_ARG;
  // S P runs on the matrix cores of the factor's dtype: 16-byte rows for S, P and the product
  const int grid = dtype == DA_BF16 ? 7 : 3;
  if ((rows | r | k) & grid) return DA_ERR_ALIGN;
  if (workspace_bytes < dion_amd_orthonormalize_sketch_workspace_bytes(batch, rows, r, k)) return DA_ERR_WORKSPACE;
  if ((uintptr_t)workspace & 255) return DA_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  char* base = static_cast<char*>(workspace);
  const size_t own = align_up(dion_amd_orthonormalize_workspace_bytes(batch, rows, r), 256);
  int* inf = info;
  if (!inf) inf = reinterpret_cast<int*>(base + align_up(da_orth_workspace_bytes(batch, rows, r), 256));
  int rc = da_fill_int(inf, batch, 0, s);
  if (rc) return rc;
  DaProfScope prof(DA_PROF_DION_ORTH, 0.0, s);
  return da_orthonormalize_sketch(P, S, out, dtype, batch, rows, r, r, k, workspace, base + own, inf, s);
}

int dion_amd_dion_step(void* const* X, const void* const* G, void* const* M, void* const* Q, int batch, int m, int n,
                       int rank, int x_dtype, int g_dtype, int m_dtype, int q_dtype, float ef_alpha, float decay,
                       float scaled_lr, float eps, int faithful, int power_iters, int* info, void* workspace,
                       size_t workspace_bytes, void* stream) {
  return dion_amd_dion_step_qr(X, G, M, Q, batch, m, n, rank, x_dtype, g_dtype, m_dtype, q_dtype, ef_alpha, decay,
                               scaled_lr, eps, faithful, power_iters, DA_QR_AUTO, info, workspace, workspace_bytes, stream);
}

int dion_amd_dion_step_qr(void* const* X, const void* const* G, void* const* M, void* const* Q, int batch, int m, int n,
                          int rank, int x_dtype, int g_dtype, int m_dtype, int q_dtype, float ef_alpha, float decay,
                          float scaled_lr, float eps, int faithful, int power_iters, int qr_method, int* info,
                          void* workspace, size_t workspace_bytes, void* stream) {
  return dion_step_impl(X, G, M, Q, batch, m, n, rank, x_dtype, g_dtype, m_dtype, q_dtype, ef_alpha, decay, scaled_lr, eps,
                        faithful, power_iters, qr_method, nullptr, 0, info, workspace, workspace_bytes, stream);
}

size_t dion_amd_dion_sketch_workspace_bytes(int batch, int m, int n, int r, int m_dtype, int sketch_k) {
  if (batch <= 0 || m <= 0 || n <= 0 || r <= 0 || sketch_k <= 0 || !dtype_ok(m_dtype)) return 0;
  return DionLayout(m, n, r, m_dtype, sketch_k).recommended(batch);
}

int dion_amd_dion_step_sketch(void* const* X, const void* const* G, void* const* M, void* const* Q, int batch, int m,
                              int n, int rank, int x_dtype, int g_dtype, int m_dtype, int q_dtype, float ef_alpha,
                              float decay, float scaled_lr, float eps, int faithful, int power_iters, const void* sketch,
                              int sketch_k, int* info, void* workspace, size_t workspace_bytes, void* stream) {
  if (!sketch || sketch_k <= 0) return DA_ERR_ARG;
  return dion_step_impl(X, G, M, Q, batch, m, n, rank, x_dtype, g_dtype, m_dtype, q_dtype, ef_alpha, decay, scaled_lr, eps,
                        faithful, power_iters, DA_QR_AUTO, sketch, sketch_k, info, workspace, workspace_bytes, stream);
}

}  // extern "C"

namespace {

int dion_step_impl(void* const* X, const void* const* G, void* const* M, void* const* Q, int batch, int m, int n,
                   int rank, int x_dtype, int g_dtype, int m_dtype, int q_dtype, float ef_alpha, float decay,
                   float scaled_lr, float eps, int faithful, int power_iters, int qr_method, const void* sketch,
                   int sketch_k, int* info, void* workspace, size_t workspace_bytes, void* stream) {
  if (qr_method < 0 || qr_method > 2) return DA_ERR_ARG;
  if (!X || !G || !M || !Q || !workspace || batch <= 0 || m <= 0 || n <= 0 || rank <= 0) return DA_ERR_ARG;
  if (power_iters < 1 || power_iters > 64) return DA_ERR_ARG;
  if (!dtype_ok(x_dtype) || !dtype_ok(g_dtype) || !dtype_ok(m_dtype) || !dtype_ok(q_dtype)) return DA_ERR_DTYPE;
  if ((m | n) & 7) return DA_ERR_ALIGN;
  if (rank > m || rank > n) return DA_ERR_ARG;
  if ((uintptr_t)workspace & 255) return DA_ERR_ALIGN;
  for (int i = 0; i < batch; ++i) {
    if (!X[i] || !G[i] || !M[i] || !Q[i]) return DA_ERR_ARG;
    if (((uintptr_t)X[i] | (uintptr_t)G[i] | (uintptr_t)M[i] | (uintptr_t)Q[i]) & 15) return DA_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const DionLayout L(m, n, rank, m_dtype, sketch ? sketch_k : 0);
  const int r = L.r;   // padded rank: pitch and logical width of Qc, P, R, Qn
  if (sketch && (sketch_k < rank || (sketch_k & 7))) return DA_ERR_ARG;
  const int chunk = L.chunk(batch, workspace_bytes);
  if (chunk < 1) return DA_ERR_WORKSPACE;
  const bool transposed = m < n;
  const int mp = L.mp, np = L.np;
  const long long mn = (long long)m * n;
  const double msz = (double)L.msz, gsz = g_dtype == DA_BF16 ? 2 : 4;

  for (int b0 = 0; b0 < batch; b0 += chunk) {
    const int cb = batch - b0 < chunk ? batch - b0 : chunk;
    // ---- carve the workspace
    char* w = static_cast<char*>(workspace);
    void** tabM = reinterpret_cast<void**>(w); w += DA_MAX_PTRS * sizeof(void*);
    void** tabX = reinterpret_cast<void**>(w); w += DA_MAX_PTRS * sizeof(void*);
    w += 2 * DA_MAX_PTRS * sizeof(void*);
    int* nonzero = reinterpret_cast<int*>(w); w += DA_MAX_PTRS * sizeof(int);
    // the orthonormaliser's status words go straight to the caller's array when there is one
    int* linfo = info ? info + b0 : reinterpret_cast<int*>(w);
    w += DA_MAX_PTRS * sizeof(int);
    w = static_cast<char*>(workspace) + L.fixed();
    char* Qc = w; w += L.qc * cb;
    char* P = w; w += L.p * cb;
    char* R = w; w += L.rb * cb;
    char* Qn = w; w += L.qn * cb;
    char* orth_ws = reinterpret_cast<char*>(align_up(reinterpret_cast<uintptr_t>(w), 256));
    char* sketch_ws = orth_ws + L.orth * cb;
    float* parts = reinterpret_cast<float*>(sketch_ws + L.sketch * cb);
    const long long sQ = (long long)(L.qc / L.msz), sP = (long long)(L.p / L.msz);

    DaPtrTable tx{}, tg{}, tm{}, tq{};
    for (int i = 0; i < cb; ++i) {
      tx.p[i] = X[b0 + i]; tg.p[i] = const_cast<void*>(G[b0 + i]); tm.p[i] = M[b0 + i]; tq.p[i] = Q[b0 + i];
    }
    int rc;
    // B = M + G inside the first P = B Q (bf16 momentum and gradients, whole 256-row tiles of B)
    const bool bq_sum = fused_bq_enabled() && da_dion_bq_sum_applicable(cb, mp, np, r, n, transposed ? 1 : 0, m_dtype, g_dtype);
    {
      DaProfScope prof(DA_PROF_DION_ELEM, bq_sum ? 0.0 : (double)mn * (2 * msz + gsz) * cb, s);
      rc = da_dion_setup(tm, tabM, tx, tabX, cb, nonzero, linfo, s);
      if (rc) return rc;
      // B = M + G, kept in M   (reference dion/dion.py:794)
      if (!bq_sum) {
        rc = da_add_grad(tm, tg, m_dtype, g_dtype, mn, cb, nonzero, s);
        if (rc) return rc;
      }
      // Q in the momentum dtype   (reference dion/dion.py:1216)
      rc = da_cast_table(tq, q_dtype, Qc, m_dtype, np, rank, r, cb, s);
      if (rc) return rc;
    }
    GemmDesc g{};
    // One power iteration is the reference's batched step (dion/dion.py:801-839); more of them repeat
    // P = orth(B Q), Q = B^T P with the unnormalised R as the next Q (dion/dion_reference.py:712-730).  The
    // all-zero / NaN guard runs in every round: between rounds it only matters for an all-zero or non-finite B.
    for (int it = 0; it < power_iters; ++it) {
      g = GemmDesc{};
      g.batch = cb; g.faithful = faithful;
      // ---- P = B Q   (reference dion/dion.py:801); B is M (mp x np) or M^T when m < n
      g.Atab = const_cast<const void* const*>(tabM); g.A = nullptr; g.lda = n; g.a_kstrided = transposed ? 1 : 0;
      g.B = it == 0 ? Qc : R; g.sB = sQ; g.ldb = r; g.b_kstrided = 1;
      g.C = P; g.sC = sP; g.ldc = r; g.c_dtype = m_dtype;
      g.M = mp; g.N = r; g.K = np;
      g.epilogue = DA_EPI_STORE; g.s0 = 0.f; g.s1 = 1.f;
      if (it == 0 && bq_sum) {
        DaProfScope prof(DA_PROF_DION_BQ, gemm_flops(g), s);
        rc = da_dion_bq_sum(tm, tg, Qc, P, sQ, sP, nonzero, cb, mp, np, r, r, n, transposed ? 1 : 0, faithful, s);
        if (rc == DA_OK && r > 256) {
          // the columns of P beyond the first 256: a plain product on the B that launch left in M
          g.B = Qc + 256 * L.msz; g.C = P + 256 * L.msz; g.N = r - 256;
          rc = da_gemm_bf16(g, s);
        }
      } else {
        rc = gemm_any(g, m_dtype, s, DA_PROF_DION_BQ);
      }
      if (rc) return rc;
      // ---- orthonormalise P   (reference dion/dion.py:822, 1267-1308)
      {
        DaProfScope prof(DA_PROF_DION_ORTH, 0.0, s);
        if (sketch) {
          // sketches: [power iteration][matrix of the bucket][sketch_k][mp] in the momentum dtype
          const char* S = static_cast<const char*>(sketch) +
                          ((size_t)it * batch + b0) * (size_t)sketch_k * mp * L.msz;
          rc = da_orthonormalize_sketch(P, S, P, m_dtype, cb, mp, r, rank, sketch_k, orth_ws, sketch_ws, linfo, s);
        } else {
          rc = da_orthonormalize(P, P, m_dtype, cb, mp, r, rank, 2, qr_method, orth_ws, linfo, s);
        }
        if (rc) return rc;
        // all-zero / NaN guard on P   (reference dion/dion.py:847, 1416-1444)
        rc = da_fix(P, nullptr, m_dtype, sP, cb, nonzero, s);
        if (rc) return rc;
      }
      // ---- R = B^T P   (reference dion/dion.py:839)
      g = GemmDesc{};
      g.batch = cb; g.faithful = faithful;
      g.Atab = const_cast<const void* const*>(tabM); g.lda = n; g.a_kstrided = transposed ? 0 : 1;
      g.B = P; g.sB = sP; g.ldb = r; g.b_kstrided = 1;
      g.C = R; g.sC = sQ; g.ldc = r; g.c_dtype = m_dtype;
      g.M = np; g.N = r; g.K = mp;
      g.epilogue = DA_EPI_STORE; g.s1 = 1.f;
      // A few output tiles with a long inner dimension (tall matrices at a low rank) leave most of the GPU idle:
      // cut the inner dimension into slices that run side by side as the groups of one launch and leave fp32
      // partial sums, which the fix-up pass that follows adds and rounds.
      const int slices = m_dtype == DA_BF16 ? btp_slices(np, r, mp, cb) : 1;
      if (slices > 1) {
        GemmDesc gs[DA_MAX_GROUPS];
        const int kslice = mp / slices;
        const long long pstride = (long long)cb * sQ;
        for (int k = 0; k < slices; ++k) {
          gs[k] = g;
          gs[k].K = kslice;
          gs[k].a_off = (long long)k * kslice * (g.a_kstrided ? n : 1);
          gs[k].B = P + (size_t)k * kslice * r * L.msz;
          gs[k].C = parts + k * pstride; gs[k].c_dtype = DA_F32; gs[k].faithful = 0;
        }
        rc = gemm_group(gs, slices, m_dtype, s, DA_PROF_DION_BTP);
        if (rc) return rc;
        DaProfScope prof(DA_PROF_DION_ELEM, 0.0, s);
        rc = da_fix_sum(parts, slices, pstride, R, Qc, m_dtype, sQ, cb, nonzero, s);
        if (rc) return rc;
      } else {
        rc = gemm_any(g, m_dtype, s, DA_PROF_DION_BTP);
        if (rc) return rc;
        DaProfScope prof(DA_PROF_DION_ELEM, 0.0, s);
        rc = da_fix(R, Qc, m_dtype, sQ, cb, nonzero, s);
        if (rc) return rc;
      }
    }  // power iterations
    // ---- error feedback, column normalisation and weight update (reference dion/dion.py:851-872)
    if (faithful && fused_update_enabled() && da_dion_ef_update_applicable(mp, np, r, m_dtype)) {
      // Q_new first (it only needs R), then both rank-r updates in one pass over M and X
      {
        DaProfScope prof(DA_PROF_DION_ELEM, 0.0, s);
        rc = da_colnorm(R, Qn, m_dtype, tq, q_dtype, np, r, rank, eps, cb, reinterpret_cast<double*>(orth_ws), s);
        if (rc) return rc;
      }
      DaProfScope prof(DA_PROF_DION_EFUPD, 4.0 * (double)mp * np * r * cb, s);
      rc = da_dion_ef_update(P, R, Qn, tm, tx, cb, mp, np, r, n, transposed ? 1 : 0, x_dtype, ef_alpha, decay,
                             scaled_lr, s);
      if (rc) return rc;
      continue;
    }
    // ---- error feedback  M <- M - (1 - mu) P R^T  (or R P^T)   (reference dion/dion.py:851-853)
    g = GemmDesc{};
    g.batch = cb; g.faithful = faithful;
    if (!transposed) { g.A = P; g.sA = sP; g.B = R; g.sB = sQ; g.M = mp; g.N = np; }
    else             { g.A = R; g.sA = sQ; g.B = P; g.sB = sP; g.M = np; g.N = mp; }
    g.lda = r; g.ldb = r; g.K = r;
    g.Ctab = tabM; g.Etab = const_cast<const void* const*>(tabM); g.ldc = n; g.lde = n; g.c_dtype = m_dtype;
    g.epilogue = DA_EPI_AXPBY; g.s0 = 1.f; g.s1 = ef_alpha;
    g.mi32 = 1;   // (the bits of the one-pass kernel)
    rc = gemm_any(g, m_dtype, s, DA_PROF_DION_EF);
    if (rc) return rc;
    // ---- Q_new = column-normalised R   (reference dion/dion.py:856, 875, 1460-1491, 1533-1561)
    {
      DaProfScope prof(DA_PROF_DION_ELEM, 0.0, s);
      // the orthonormaliser is done with its fp64 scratch: reuse its head for the column sums
      rc = da_colnorm(R, Qn, m_dtype, tq, q_dtype, np, r, rank, eps, cb, reinterpret_cast<double*>(orth_ws), s);
      if (rc) return rc;
    }
    // ---- X <- (1 - lr wd) X - scaled_lr P Q_new^T  (or Q_new P^T)   (reference dion/dion.py:865-872)
    g = GemmDesc{};
    g.batch = cb; g.faithful = faithful;
    if (!transposed) { g.A = P; g.sA = sP; g.B = Qn; g.sB = sQ; g.M = mp; g.N = np; }
    else             { g.A = Qn; g.sA = sQ; g.B = P; g.sB = sP; g.M = np; g.N = mp; }
    g.lda = r; g.ldb = r; g.K = r;
    g.Ctab = tabX; g.Etab = const_cast<const void* const*>(tabX); g.ldc = n; g.lde = n; g.c_dtype = x_dtype;
    g.epilogue = DA_EPI_AXPBY; g.s0 = decay; g.s1 = -scaled_lr;
    g.mi32 = 1;
    rc = gemm_any(g, m_dtype, s, DA_PROF_DION_UPD);
    if (rc) return rc;
  }
  return DA_OK;
}

}  // namespace
