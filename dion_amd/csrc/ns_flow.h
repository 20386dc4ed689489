// Host-side interface of the persistent Newton-Schulz kernel (ns_flow.hip): all iterations of many small wide
// matrices in one launch.
#pragma once
#include "common.h"

constexpr int DA_FLOW_MAX_STEPS = 8;      // Newton-Schulz iterations per launch
constexpr int DA_FLOW_CTR_STRIDE = 32;    // ints of control memory per matrix (3 counters per iteration)

// One bucket of `cnt` same-shape wide matrices (mw <= nw, both multiples of 256) in bf16 working buffers:
// x0, x1: [cnt][mw][ldx] (x0 holds the normalised input, the result ends up in x0 or x1: whichever is not the
// input of the last iteration), a, b: [cnt][mw][lda]; sx / sa: elements between consecutive matrices.
// ctl: da_ns_flow_ctl_bytes(cnt) bytes of device memory for the launch's counters (cleared by the launch itself).
struct DaNsFlowGroup {
  char *x0, *x1, *a, *b;
  long long sx, sa;
  int mw, nw, ldx, lda, cnt;
  int* ctl;
  // upd_tab != null: the last iteration's X' is not stored but updates the bf16 weights upd_tab[b] in place (see GemmDesc)
  void* const* upd_tab;
  int upd_dtype, upd_ld, upd_transposed;
  float upd_decay, upd_step;
};

size_t da_ns_flow_ctl_bytes(int cnt);
// Whether the persistent kernel runs these groups (shapes on the 256 grid and, unless forced, a workload it is
// faster on: many small matrices that deal evenly to the eight queues).
bool da_ns_flow_applicable(const DaNsFlowGroup* g, int n, int steps, int faithful);
int da_ns_flow(const DaNsFlowGroup* g, int n, const float* coeffs, int steps, int faithful, hipStream_t s);
// Device word that is non-zero after a launch that gave up (a wait beyond the spin limit): results are then invalid.
const int* da_ns_flow_status_word(const DaNsFlowGroup* g);
// mode: -1 automatic (DION_AMD_NS_FLOW in the environment, else by workload), 0 never, 1 whenever the shapes
// allow, 2 the same with an L2 write-back after every tile.  fail (test hook): launches start with the status word set.
void da_ns_flow_set_mode(int mode);
void da_ns_flow_set_fail(int on);
void da_ns_flow_set_spin_limit(long long ticks);
// Measurement hook: while enabled, every tile of a launch records the 100 MHz counter at its start, when its
// dependency was met, after its K loop and after its result was published, plus (queue << 48 | phase << 32 | ticket)
// and (XCD << 32 | HW_ID).  `read` waits for the device and copies up to max_tiles records (six 64-bit words each) of
// the most recent traced launch to host memory.
void da_ns_flow_trace_enable(int on);
int da_ns_flow_trace_read(void* host_dst, int max_tiles, int* tiles);
