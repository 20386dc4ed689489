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
// The same with the divisor formed inside the launch from the partial sums of squares (`tiles` per matrix; what
// da_norm_finish would have written: same order of summation, same roundings).  partials == null: read `divisor`.
int da_normalize_from_partials(void* wide, int w_dtype, long long per_matrix, int batch, const float* divisor,
                               const float* partials, int tiles, float eps, hipStream_t s);
int da_unstage(const DaUnstage& d, hipStream_t s);
// Up to DA_MAX_UPLOADS pointer tables in one launch: dst[k][i] = t[k].p[i] for i < n[k]; and the same tables as the
// target of a conditional poisoning (numel[k] contiguous elements per matrix of table k).
constexpr int DA_MAX_UPLOADS = 6;
struct DaPtrUploads {
  DaPtrTable t[DA_MAX_UPLOADS];
  void** dst[DA_MAX_UPLOADS];
  int n[DA_MAX_UPLOADS];
};
struct DaPoisonShape {
  long long numel[DA_MAX_UPLOADS];
  int f32;
};
int da_upload_ptrs_multi(const DaPtrUploads& u, int count, hipStream_t s);
int da_poison_multi_if(const DaPtrUploads& u, int count, const DaPoisonShape& sh, const int* flag, hipStream_t s);
// dst[i] = t.p[i] for i < n <= DA_MAX_PTRS: a table of per-matrix pointers in device memory
int da_upload_ptrs(const DaPtrTable& t, void** dst, int n, hipStream_t s);
// If *flag != 0 when the kernel runs, every element of the n matrices (numel contiguous elements each) becomes NaN.
int da_poison_if(const DaPtrTable& t, int n, long long numel, int dtype, const int* flag, hipStream_t s);
