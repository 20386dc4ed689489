// All Newton-Schulz iterations of many small matrices as ONE persistent launch.
//
//   per iteration and matrix:  A = X X^T ;  B = b A + c A A ;  X' = a X + B X      (reference dion/muon.py:638-643)
//
// Launched product by product, a step over many small matrices (GPT-small: 48 x 768^2, 24 x 768x3072) loses a
// third of its time to the ends of launches: 1296 tiles on 256 compute units are 5.06 rounds that cost 6, a
// product is as long as its longest tile, and between two launches the GPU drains.  Here a workgroup per compute
// unit takes tile after tile of ALL products of ALL iterations from a queue, and a tile starts as soon as the
// product it reads is complete for ITS matrix: per matrix and product a counter in device memory counts finished
// tiles.  No grid-wide synchronisation anywhere.
//
// Queues and caches.  The eight XCDs have an L2 each, and data written through one L2 is visible to readers behind
// another only after a write-back there and an invalidation here.  So every matrix belongs to one of eight
// queues, a queue is worked on by the workgroups of ONE XCD only -- the first XCD that takes a ticket from it owns
// it, which is the queue's own XCD unless that one has no workgroup of this launch at all -- and all tiles of a
// matrix, producers and consumers alike, meet in the same L2: a finished tile needs its stores acknowledged (they
// are then in the L2) before its counter moves, a starting tile drops its compute unit's L1 lines, and nothing
// else.  Ticket and counter words themselves are agent-scope atomics.  (`strict` mode adds the L2 write-back to
// every finished tile; it is the memory model's own recipe for any placement and serves as the cross-check.)
//
// Order.  Tickets of a queue run (iteration, product, matrix, tile); matrices are dealt to the queues round-robin
// in the order given (the caller sorts the groups by cost, costliest first); X X^T takes the groups in that order,
// the two products behind it in the opposite one.  The order is topological -- a tile's producers hold smaller
// tickets of the same queue -- so a waiting workgroup only ever waits for workgroups that are running: no deadlock,
// whatever the placement and however many workgroups are resident.  Every wait is bounded all the same: after
// `spin_limit` ticks of the 100 MHz counter a workgroup sets the status word and every workgroup leaves at its
// next ticket; the caller poisons its results with the status word (da_unstage).
//
// The tile itself -- K loop, rounding-faithful epilogue, mirrored store of symmetric results -- is the code of the
// batched GEMM kernel (gemm_bf16_tile.h), so the results are the same bits.
#include "ns_flow.h"
#include "gemm_bf16_tile.h"
#include <cstdlib>

namespace {

typedef Cfg<256, 2, 4> Big;
constexpr int BT = 256;
constexpr int NQ = 8;                      // queues = XCDs
constexpr unsigned OWNER_SHIFT = 28;       // ticket word: (owner XCD + 1) << 28 | next index
constexpr unsigned INDEX_MASK = (1u << OWNER_SHIFT) - 1;

struct FlowGroupDev {
  char *x0, *x1, *a, *b;
  long long sx, sa;          // elements between consecutive matrices
  int* counters;             // [cnt][DA_FLOW_CTR_STRIDE]
  void* const* upd_tab;      // weights updated by the last iteration's X' (or null: X' is stored)
  float upd_decay, upd_step;
  int upd_dtype, upd_ld, upd_transposed;
  int mw, nw, ldx, lda;
  int cnt, first;            // matrices; index of the first one in the dealing order
  int tm, tn;                // tiles per side
};

struct FlowArgs {
  FlowGroupDev g[DA_MAX_GROUPS];
  float coeffs[3 * DA_FLOW_MAX_STEPS];
  unsigned* tickets;         // [NQ]
  int* status;
  unsigned long long spin_limit;
  unsigned long long* trace;     // measurement hook: six words per finished tile, or null
  unsigned* trace_count;
  int trace_cap;
  int ngroups, steps, faithful, strict;
};

__device__ __forceinline__ int ceil8(int x) { return (x + 7) >> 3; }   // x >= -7

struct Item { int it, p, g, b, t; bool valid; };

// ticket `t` of queue `q` -> (iteration, product, group, matrix, tile); all scalar arithmetic, no indexed arrays
__device__ __forceinline__ Item decode(const FlowArgs& a, int q, int t) {
  int p_sym = 0, p_ax = 0;
#pragma unroll
  for (int g = 0; g < DA_MAX_GROUPS; ++g) {
    if (g < a.ngroups) {
      const FlowGroupDev& G = a.g[g];
      const int nq = ceil8(G.first + G.cnt - q) - ceil8(G.first - q);
      p_sym += nq * (G.tm * (G.tm + 1) / 2);
      p_ax += nq * (G.tm * G.tn);
    }
  }
  Item r{};
  const int per_it = 2 * p_sym + p_ax;
  r.valid = per_it > 0 && t < per_it * a.steps;
  if (!r.valid) return r;
  r.it = t / per_it;
  int rem = t - r.it * per_it;
  r.p = 0;
  if (rem >= p_sym) { rem -= p_sym; r.p = 1; }
  if (r.p == 1 && rem >= p_sym) { rem -= p_sym; r.p = 2; }
  r.g = 0;
  int per = 1, first = 0;
  bool found = false;
  // X X^T takes the groups costliest first (their tiles are the long ones: K is the matrix's long side); the two
  // products behind it take them cheapest first, so that the tickets that follow X X^T belong to matrices whose
  // X X^T was over first, and the costly group's tiles are requested when its long tiles have had time to finish
#pragma unroll
  for (int i = 0; i < DA_MAX_GROUPS; ++i) {
    if (i < a.ngroups && !found) {
      const int g = r.p == 0 ? i : a.ngroups - 1 - i;
      const FlowGroupDev& G = a.g[g];
      const int nq = ceil8(G.first + G.cnt - q) - ceil8(G.first - q);
      const int tiles = r.p == 2 ? G.tm * G.tn : G.tm * (G.tm + 1) / 2;
      if (rem < nq * tiles || i + 1 == a.ngroups) {
        found = true;
        r.g = g; per = tiles; first = G.first;
      } else {
        rem -= nq * tiles;
      }
    }
  }
  const int k = rem / per;
  r.t = rem - k * per;
  r.b = ((q - first) & 7) + 8 * k;     // the k-th matrix of the group whose dealing index is q modulo 8
  return r;
}

__device__ __forceinline__ unsigned long long now_ticks() { return __builtin_amdgcn_s_memrealtime(); }

// Next ticket of queue q for a workgroup on XCD `xcd`, or -1: the queue is used up or belongs to another XCD.
// `owned`: this workgroup has taken a ticket of the queue before (the owner field is then known to be `xcd`).
__device__ __forceinline__ int take_ticket(unsigned* word, int xcd, int total, bool owned) {
  const unsigned me = (unsigned)(xcd + 1);
  if (!owned) {
    unsigned cur = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((cur >> OWNER_SHIFT) == 0) {
      unsigned expect = 0;
      if (__hip_atomic_compare_exchange_strong(word, &expect, (me << OWNER_SHIFT) | 1u, __ATOMIC_RELAXED,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
        return 0;
      cur = expect;          // somebody else's claim went first
    }
    if ((cur >> OWNER_SHIFT) != me) return -1;
  }
  const unsigned old = __hip_atomic_fetch_add(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned idx = old & INDEX_MASK;
  return idx < (unsigned)total ? (int)idx : -1;
}

__global__ __launch_bounds__(Big::NT) void ns_flow_kernel(FlowArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  __shared__ int sh_ticket[2];
  __shared__ int sh_abort, sh_wait;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = wave_uniform(tid >> 6);
  const int wm = wave / Big::WGN, wn = wave % Big::WGN;
  const int xcd = (int)(__builtin_amdgcn_s_getreg(20 | (3 << 11)) & 7u);   // XCC_ID
  if (tid == 0) sh_abort = 0;
  const bool trace = a.trace != nullptr;

  for (int qi = 0; qi < NQ; ++qi) {
    const int q = (xcd + qi) & (NQ - 1);
    int total = 0;             // tickets of this queue
    for (int g = 0; g < a.ngroups; ++g) {
      const FlowGroupDev& G = a.g[g];
      const int n = ceil8(G.first + G.cnt - q) - ceil8(G.first - q);
      total += n * (G.tm * (G.tm + 1) + G.tm * G.tn);
    }
    total *= a.steps;
    if (total <= 0) continue;
    int slot = 0;
    // A finished tile is published -- its counter moved -- one tile late: under the first stage of the next tile's K
    // loop, behind whose barrier every wavefront's stores are acknowledged anyway.  Waiting for them right after the
    // epilogue costs 2-3 us per tile.  (Before a workgroup waits for a dependency it publishes what it holds: the
    // tile it waits for must not be its own.)
    int* pend = nullptr;
    auto publish = [&]() {
      if (pend != nullptr && tid == 0) {
        if (a.strict) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");   // L2 write-back: visible behind any L2
        __hip_atomic_fetch_add(pend, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      pend = nullptr;
    };
    auto flush = [&]() {
      if (pend != nullptr) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        publish();
      }
    };
    if (tid == 0) sh_ticket[0] = take_ticket(a.tickets + q, xcd, total, false);
    while (true) {
      __syncthreads();
      const int t = wave_uniform(sh_ticket[slot]);
      if (t < 0) {             // next queue
        flush();
        break;
      }
      unsigned long long ts[4] = {0, 0, 0, 0};
      if (trace) ts[0] = now_ticks();
      Item w = decode(a, q, t);
      // (the divisions run on the vector unit: back into scalar registers, or every address below is per lane)
      w.it = wave_uniform(w.it); w.p = wave_uniform(w.p); w.g = wave_uniform(w.g);
      w.b = wave_uniform(w.b); w.t = wave_uniform(w.t);
      const FlowGroupDev& G = a.g[w.g];
      int* ctr = G.counters + (long long)w.b * DA_FLOW_CTR_STRIDE;
      const int phase = w.it * 3 + w.p;
      const int tsym = G.tm * (G.tm + 1) / 2;
      // ---- wait until the product this tile reads is complete for its matrix
      const int want = w.p == 0 ? G.tm * G.tn : tsym;   // X X^T reads the previous iteration's X'
      const int* dep = ctr + phase - 1;
      if (tid == 0)
        sh_wait = phase > 0 && __hip_atomic_load(dep, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want ? 1 : 0;
      __syncthreads();
      if (wave_uniform(sh_wait) != 0) {
        flush();
        if (tid == 0) {
          const unsigned long long t0 = now_ticks();
          while (__hip_atomic_load(dep, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
            __builtin_amdgcn_s_sleep(4);
            if (now_ticks() - t0 > a.spin_limit ||
                __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
              // give the launch up: whoever waits next sees the status word and leaves as well
              __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              sh_abort = 1;
              break;
            }
          }
        }
        __syncthreads();
        if (wave_uniform(sh_abort) != 0) return;
      }
      // drop this compute unit's L1 lines: the buffers are rewritten from iteration to iteration.  (An agent-scope
      // acquire would do that too, but it also drops what this XCD's L2 holds for the other 31 compute units.)
      if (a.strict) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      else asm volatile("buffer_inv sc0" ::: "memory");
      if (trace) ts[1] = now_ticks();

      // ---- the tile
      const float ca = a.coeffs[3 * w.it], cb = a.coeffs[3 * w.it + 1], cc = a.coeffs[3 * w.it + 2];
      char* xcur = (w.it & 1) ? G.x1 : G.x0;
      char* xnext = (w.it & 1) ? G.x0 : G.x1;
      GemmDesc d{};
      d.batch = 1; d.c_dtype = DA_BF16; d.faithful = a.faithful;
      int ti, tj;
      if (w.p == 2) {
        ti = w.t / G.tn;
        tj = w.t - ti * G.tn;
      } else {
        ti = 0;
        int rem = w.t, len = G.tm;
        while (rem >= len) { rem -= len; ++ti; --len; }
        tj = ti + rem;
      }
      ti = wave_uniform(ti);
      tj = wave_uniform(tj);
      const int m0 = ti * BT, n0 = tj * BT;
      int next = -1;           // (thread 0) the next ticket
      Big::acc_t acc[Big::TMI][Big::TNJ];
      const bf16_t *Aop, *Bop;
      if (w.p == 0) {
        Aop = Bop = reinterpret_cast<const bf16_t*>(xcur) + (long long)w.b * G.sx;
        d.C = G.a + (long long)w.b * G.sa * 2;
        d.lda = G.ldx; d.ldb = G.ldx; d.ldc = G.lda;
        d.M = G.mw; d.N = G.mw; d.K = G.nw;
        d.symmetric = 1; d.epilogue = DA_EPI_STORE;
      } else if (w.p == 1) {
        Aop = Bop = reinterpret_cast<const bf16_t*>(G.a) + (long long)w.b * G.sa;
        d.C = G.b + (long long)w.b * G.sa * 2;
        d.E = Aop;
        d.lda = G.lda; d.ldb = G.lda; d.ldc = G.lda; d.lde = G.lda;
        d.M = G.mw; d.N = G.mw; d.K = G.mw;
        d.symmetric = 1; d.epilogue = DA_EPI_AXPBY;
      } else {
        Aop = reinterpret_cast<const bf16_t*>(G.b) + (long long)w.b * G.sa;
        Bop = reinterpret_cast<const bf16_t*>(xcur) + (long long)w.b * G.sx;
        d.C = xnext + (long long)w.b * G.sx * 2;
        d.E = Bop;
        d.lda = G.lda; d.ldb = G.ldx; d.ldc = G.ldx; d.lde = G.ldx;
        d.M = G.mw; d.N = G.nw; d.K = G.mw;
        d.b_kstrided = 1; d.epilogue = DA_EPI_AXPBY;
        if (G.upd_tab != nullptr && w.it + 1 == a.steps) {
          d.upd_tab = G.upd_tab + w.b; d.upd_dtype = G.upd_dtype; d.upd_ld = G.upd_ld;
          d.upd_transposed = G.upd_transposed; d.upd_decay = G.upd_decay; d.upd_step = G.upd_step;
        }
      }
      // epilogue scalars, C = s0 E + s1 acc.  (As selects on purpose: assigned inside the three branches above, hipcc 7.2
      // passed the polynomial's b as s0 of X' = aX + BX; the bit-level tests against the product launches cover it.)
      d.s0 = w.p == 2 ? ca : (w.p == 1 ? cb : 0.f);
      d.s1 = w.p == 1 ? cc : 1.f;
      if (w.p == 2) gemm_tile_k_loop<Big, false, true, DA_LOOP_INTERIOR>(acc, d, Aop, Bop, d.K, m0, n0, lds, tid, lane, wave, wm, wn, publish);
      else gemm_tile_k_loop<Big, false, false, DA_LOOP_INTERIOR>(acc, d, Aop, Bop, d.K, m0, n0, lds, tid, lane, wave, wm, wn, publish, ti == tj);
      if (trace) ts[2] = now_ticks();
      // the next ticket is requested before the epilogue, which hides its latency
      if (tid == 0) next = take_ticket(a.tickets + q, xcd, total, true);
      // the epilogue forms this kernel needs, and no others (every form compiled in costs registers here): bf16
      // results, rounding-faithful; X X^T stores acc, the polynomial and X' combine with E, the last X' may update
      // bf16 weights instead of being stored
      const bool mirror = ti != tj;
#define DA_FLOW_EPI(SYMM, HE, ONE, U) \
  epilogue_impl<Big, SYMM, true, false, HE, true, ONE, U, false>(acc, d, lds, 0, SYMM && mirror, m0, n0, wave, lane, wm, wn)
      if (w.p == 0) DA_FLOW_EPI(true, false, true, 0);
      else if (w.p == 1) DA_FLOW_EPI(true, true, false, 0);
      else if (d.upd_tab == nullptr) DA_FLOW_EPI(false, true, true, 0);
      else if (d.upd_transposed) DA_FLOW_EPI(false, true, true, 2);
      else DA_FLOW_EPI(false, true, true, 1);
#undef DA_FLOW_EPI
      // ---- to be published under the next tile
      pend = ctr + phase;
      if (tid == 0) {
        sh_ticket[slot ^ 1] = next;
        if (trace) {
          // (queue, ticket) -> taken, dependency met, K loop done, epilogue done; product and iteration
          const unsigned rec = __hip_atomic_fetch_add(a.trace_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (rec < (unsigned)a.trace_cap) {
            unsigned long long* o = a.trace + (size_t)rec * 6;
            o[0] = ts[0]; o[1] = ts[1]; o[2] = ts[2]; o[3] = now_ticks();
            o[4] = ((unsigned long long)q << 48) | ((unsigned long long)phase << 32) | (unsigned)t;
            o[5] = ((unsigned long long)xcd << 32) | __builtin_amdgcn_s_getreg(4 | (31 << 11));
          }
        }
      }
      slot ^= 1;
    }
    // thread 0 rewrites sh_ticket for the next queue: not before every wavefront has read this queue's last one
    __syncthreads();
  }
}

// clears the counters of up to DA_MAX_GROUPS groups, the ticket words and the status word (`preset`: test hook)
struct ResetArgs {
  int* p[DA_MAX_GROUPS];
  int n[DA_MAX_GROUPS];
  unsigned* tickets;
  int* status;
  unsigned* trace_count;
  int preset;
};
__global__ __launch_bounds__(256) void ns_flow_reset_kernel(ResetArgs r) {
  const int g = blockIdx.y;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < r.n[g]; i += gridDim.x * 256) r.p[g][i] = 0;
  if (g == 0 && blockIdx.x == 0) {
    if (threadIdx.x < NQ) r.tickets[threadIdx.x] = 0u;
    if (threadIdx.x == NQ) *r.status = r.preset;
    if (threadIdx.x == NQ + 1 && r.trace_count) *r.trace_count = 0u;
  }
}

// Measurement hook: time line of the tiles of the most recent traced launch.
constexpr int FLOW_TRACE_CAP = 1 << 16;
__device__ unsigned long long flow_trace[6 * FLOW_TRACE_CAP];
__device__ unsigned flow_trace_count;
std::atomic<bool> g_flow_trace{false};

std::atomic<int> g_flow_mode{-1};          // -1: automatic, 0: never, 1: whenever the shapes allow, 2: same, strict
std::atomic<int> g_flow_fail{0};           // test hook: the launch starts with the status word set
std::atomic<long long> g_flow_spin{-1};    // ticks of the 100 MHz counter; -1: default

double tile_cost(int stages, int product) {
  // microseconds, from the tile time lines of the batched kernel: 1.7 per 64-deep stage, epilogue, ticket + wait
  const double epi = product == 2 ? 5.5 : (product == 1 ? 4.5 : 4.0);
  return 1.7 * stages + epi + 1.0;
}

}  // namespace

void da_ns_flow_trace_enable(int on) { g_flow_trace.store(on != 0, std::memory_order_relaxed); }
int da_ns_flow_trace_read(void* dst, int max_tiles, int* tiles) {
  if (!dst || !tiles || max_tiles <= 0) return DA_ERR_ARG;
  DA_HIP_CHECK(hipDeviceSynchronize());
  unsigned n = 0;
  DA_HIP_CHECK(hipMemcpyFromSymbol(&n, HIP_SYMBOL(flow_trace_count), sizeof(n)));
  if (n > (unsigned)FLOW_TRACE_CAP) n = FLOW_TRACE_CAP;
  if (n > (unsigned)max_tiles) n = (unsigned)max_tiles;
  if (n) DA_HIP_CHECK(hipMemcpyFromSymbol(dst, HIP_SYMBOL(flow_trace), (size_t)n * 6 * sizeof(unsigned long long)));
  *tiles = (int)n;
  return DA_OK;
}
void da_ns_flow_set_mode(int mode) { g_flow_mode.store(mode, std::memory_order_relaxed); }
void da_ns_flow_set_fail(int on) { g_flow_fail.store(on, std::memory_order_relaxed); }
void da_ns_flow_set_spin_limit(long long ticks) { g_flow_spin.store(ticks, std::memory_order_relaxed); }

size_t da_ns_flow_ctl_bytes(int cnt) { return (size_t)cnt * DA_FLOW_CTR_STRIDE * sizeof(int) + 256; }

bool da_ns_flow_applicable(const DaNsFlowGroup* g, int n, int steps, int faithful) {
  if (!faithful) return false;   // (the kernel carries the rounding-faithful epilogues only)
  int mode = g_flow_mode.load(std::memory_order_relaxed);
  if (mode < 0) {
    static const int env = [] { const char* e = getenv("DION_AMD_NS_FLOW"); return e ? atoi(e) : -1; }();
    mode = env;
  }
  if (mode == 0) return false;
  if (n < 1 || n > DA_MAX_GROUPS || steps < 1 || steps > DA_FLOW_MAX_STEPS) return false;
  long long nmat = 0;
  double load[NQ] = {0};
  double par_min = 1e30;
  for (int i = 0; i < n; ++i) {
    const DaNsFlowGroup& G = g[i];
    if (G.cnt < 1 || G.mw % BT || G.nw % BT || G.mw > G.nw) return false;
    // 32-bit byte offsets inside a tile's operand panels (as for the batched kernel's direct-to-LDS loop)
    if ((long long)G.mw * G.ldx * 2 >= (1LL << 32) || (long long)G.mw * G.lda * 2 >= (1LL << 32)) return false;
    const int tm = G.mw / BT, tn = G.nw / BT, tsym = tm * (tm + 1) / 2;
    const double cost = tsym * tile_cost(G.nw / 64, 0) + tsym * tile_cost(G.mw / 64, 1) + tm * tn * tile_cost(G.mw / 64, 2);
    for (int j = 0; j < G.cnt; ++j) load[(nmat + j) & 7] += cost;
    nmat += G.cnt;
    if (nmat * DA_FLOW_CTR_STRIDE > 0x7fffffffLL) return false;
  }
  if (mode >= 1) return true;
  // automatic: many small matrices, evenly dealt, each queue with enough tiles of one product to keep an XCD's
  // 32 compute units busy
  if (nmat < 16) return false;
  double mx = 0, sum = 0;
  for (int q = 0; q < NQ; ++q) { mx = load[q] > mx ? load[q] : mx; sum += load[q]; }
  if (mx > 1.06 * sum / NQ) return false;
  for (int q = 0; q < NQ; ++q) {
    double tiles = 0;
    long long s = 0;
    for (int i = 0; i < n; ++i) {
      const int tm = g[i].mw / BT;
      const int nq = (int)(((s + g[i].cnt - q + 7) >> 3) - ((s - q + 7) >> 3));
      tiles += (double)nq * tm * (tm + 1) / 2;
      s += g[i].cnt;
    }
    par_min = tiles < par_min ? tiles : par_min;
  }
  if (par_min < 40) return false;
  // large matrices fill the GPU product by product and lose little at the ends of launches; they also want the
  // whole GPU on one matrix for their panels' sake
  for (int i = 0; i < n; ++i)
    if ((long long)g[i].mw * g[i].nw > 1024LL * 4096) return false;
  return true;
}

int da_ns_flow(const DaNsFlowGroup* g, int n, const float* coeffs, int steps, int faithful, hipStream_t s) {
  if (!g || !coeffs || n < 1 || n > DA_MAX_GROUPS || steps < 1 || steps > DA_FLOW_MAX_STEPS || !faithful) return DA_ERR_ARG;
  FlowArgs a{};
  ResetArgs r{};
  int first = 0;
  for (int i = 0; i < n; ++i) {
    const DaNsFlowGroup& G = g[i];
    if (!G.x0 || !G.x1 || !G.a || !G.b || !G.ctl || G.cnt < 1) return DA_ERR_ARG;
    if (G.upd_tab && G.upd_dtype != DA_BF16) return DA_ERR_DTYPE;   // (weights of another dtype: the caller's own pass)
    if (G.mw % BT || G.nw % BT || G.mw > G.nw || (G.ldx & 7) || (G.lda & 7) || (G.sx & 7) || (G.sa & 7)) return DA_ERR_ALIGN;
    FlowGroupDev& D = a.g[i];
    D.x0 = G.x0; D.x1 = G.x1; D.a = G.a; D.b = G.b;
    D.sx = G.sx; D.sa = G.sa;
    D.counters = G.ctl;
    D.upd_tab = G.upd_tab; D.upd_dtype = G.upd_dtype; D.upd_ld = G.upd_ld; D.upd_transposed = G.upd_transposed;
    D.upd_decay = G.upd_decay; D.upd_step = G.upd_step;
    D.mw = G.mw; D.nw = G.nw; D.ldx = G.ldx; D.lda = G.lda;
    D.cnt = G.cnt; D.first = first;
    D.tm = G.mw / BT; D.tn = G.nw / BT;
    r.p[i] = G.ctl; r.n[i] = G.cnt * DA_FLOW_CTR_STRIDE;
    first += G.cnt;
  }
  // the ticket and status words live behind the counters of the first group
  int* tail = g[0].ctl + (size_t)g[0].cnt * DA_FLOW_CTR_STRIDE;
  a.tickets = reinterpret_cast<unsigned*>(tail);
  a.status = tail + NQ;
  r.tickets = a.tickets; r.status = a.status;
  r.preset = g_flow_fail.load(std::memory_order_relaxed) ? 1 : 0;
  for (int i = 0; i < 3 * steps; ++i) a.coeffs[i] = coeffs[i];
  a.ngroups = n; a.steps = steps; a.faithful = faithful;
  int mode = g_flow_mode.load(std::memory_order_relaxed);
  if (mode < 0) {
    static const int env = [] { const char* e = getenv("DION_AMD_NS_FLOW"); return e ? atoi(e) : -1; }();
    mode = env;
  }
  a.strict = mode == 2;
  const long long spin = g_flow_spin.load(std::memory_order_relaxed);
  a.spin_limit = spin >= 0 ? (unsigned long long)spin : 200000000ull;   // 2 s of the 100 MHz counter

  if (g_flow_trace.load(std::memory_order_relaxed)) {
    void *tp = nullptr, *cp = nullptr;
    DA_HIP_CHECK(hipGetSymbolAddress(&tp, HIP_SYMBOL(flow_trace)));
    DA_HIP_CHECK(hipGetSymbolAddress(&cp, HIP_SYMBOL(flow_trace_count)));
    a.trace = static_cast<unsigned long long*>(tp);
    a.trace_count = static_cast<unsigned*>(cp);
    a.trace_cap = FLOW_TRACE_CAP;
    r.trace_count = a.trace_count;
  }
  hipLaunchKernelGGL(ns_flow_reset_kernel, dim3(8, (unsigned)n), dim3(256), 0, s, r);
  int rc = da_launch_status();
  if (rc) return rc;
  constexpr int smem = 2 * (Tile<BT, false>::bytes + Tile<BT, false>::bytes);
  static DaOncePerDevice configured;
  rc = configured.run([&]() -> int {
    DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(ns_flow_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return DA_OK;
  });
  if (rc) return rc;
  hipLaunchKernelGGL(ns_flow_kernel, dim3((unsigned)da_cu_count()), dim3(Big::NT), smem, s, a);
  return da_launch_status();
}

const int* da_ns_flow_status_word(const DaNsFlowGroup* g) {
  return g[0].ctl + (size_t)g[0].cnt * DA_FLOW_CTR_STRIDE + NQ;
}
