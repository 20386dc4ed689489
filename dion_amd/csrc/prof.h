// Optional per-launch timing with HIP events on the launch stream (measurement only;
// disabled by default, zero cost when disabled apart from one branch per launch).
#pragma once
#include <hip/hip_runtime.h>

enum DaProfKind {
  DA_PROF_NS_SYRK = 0,    // A = X X^T
  DA_PROF_NS_POLY = 1,    // B = b A + c A A
  DA_PROF_NS_AXPY = 2,    // X' = a X + B X
  DA_PROF_STAGE = 3,      // momentum / cast -> wide working matrix (+ sum of squares)
  DA_PROF_NORMALIZE = 4,  // X / (||X|| + eps)
  DA_PROF_UNSTAGE = 5,    // weight update / store
  DA_PROF_GEMM = 6,       // general GEMM entry point
  DA_PROF_DION_BQ = 7,    // P = B Q
  DA_PROF_DION_BTP = 8,   // R = B^T P
  DA_PROF_DION_EF = 9,    // M <- B - (1-mu) P R^T
  DA_PROF_DION_UPD = 10,  // X <- (1 - lr wd) X - lr' P Q^T
  DA_PROF_DION_ORTH = 11, // orthonormalisation of P (all of its launches)
  DA_PROF_DION_ELEM = 12, // B = M + G, column norms, guards
  DA_PROF_SCALAR_OPT = 13,// fused Lion / AdamW pass over non-matrix parameters
  DA_PROF_DION_EFUPD = 14,// error feedback and weight update in one pass
  DA_PROF_NS_FLOW = 15,   // all Newton-Schulz iterations of a set of buckets in one persistent launch
  DA_PROF_KINDS = 16
};

struct DaProfScope {
  int slot;
  hipStream_t s;
  DaProfScope(int kind, double work, hipStream_t stream);
  ~DaProfScope();
};
