// Host-side launch descriptors for the HBM-bound passes (see elementwise.hip).
#pragma once
#include "common.h"

#define DA_MAX_PTRS 64  // matrices per launch: pointer tables travel as kernel arguments

struct DaPtrTable {
  void* p[DA_MAX_PTRS];
};

struct DaStage {
  DaPtrTable g;      // source matrices (rows x cols, row pitch ld)
  DaPtrTable mom;    // momentum buffers (contiguous rows x cols), Muon mode only
  void* wide;        // [batch][min(rows,cols)][ldw] working matrices, max(rows,cols) columns used
  float* partials;   // [batch][da_stage_tiles(rows, cols)]
  int batch, rows, cols, ld;
  int ldw;           // row pitch of the working matrices (elements, multiple of 8, >= max(rows,cols))
  int g_dtype, m_dtype, w_dtype;
  float mu;
  int nesterov;
  int muon;
  // Stand-alone momentum pass (no Newton-Schulz behind it): each result keeps the source orientation and goes
  // to its own matrix wtab.p[b] (rows x cols, contiguous) instead of the batch `wide`; no partial sums.
  int use_wtab;
  DaPtrTable wtab;
};

struct DaUnstage {
  DaPtrTable x;      // destinations (rows x cols, row pitch ld)
  const void* wide;
  int batch, rows, cols, ld;
  int ldw;           // row pitch of the working matrices
  int x_dtype, w_dtype;
  float decay, step;
  int muon;
  // Stand-alone weight update: the orthogonalised matrices are wtab.p[b] (rows x cols, contiguous, source
  // orientation) instead of the batch `wide`.
  int use_wtab;
  DaPtrTable wtab;
  // Optional device word: if it is non-zero when the kernel runs, the working matrices are invalid (the launch that
  // made them gave up) and every result element is written as NaN.
  const int* poison;
};

int da_stage_tiles(int rows, int cols);
int da_stage_wide(const DaStage& d, hipStream_t s);
int da_norm_finish(const float* partials, int tiles, int batch, float eps, int bf16_mode, float* divisor,
                   hipStream_t s);
int da_normalize(void* wide, int w_dtype, long long per_matrix, int batch, const float* divisor, hipStream_t s);
int da_unstage(const DaUnstage& d, hipStream_t s);
// dst[i] = t.p[i] for i < n <= DA_MAX_PTRS: a table of per-matrix pointers in device memory
int da_upload_ptrs(const DaPtrTable& t, void** dst, int n, hipStream_t s);
// If *flag != 0 when the kernel runs, every element of the n matrices (numel contiguous elements each) becomes NaN.
int da_poison_if(const DaPtrTable& t, int n, long long numel, int dtype, const int* flag, hipStream_t s);
