// Ceiling probes (measurement only; no counterpart in the reference): what the two engines a bf16 GEMM's K loop
// leans on deliver on this GPU when nothing else is in their way.
//
//   matrix cores : every wavefront issues v_mfma_f32_32x32x16_bf16 back to back on eight independent accumulators
//                  with operands held in registers (random bf16 values: the power a matrix core draws, and with it
//                  the clock the chip sustains, depends on the data), two wavefronts per SIMD as in the GEMM kernel.
//                  (A second form issues v_mfma_f32_16x16x32_bf16 on sixteen accumulators: the same flops per pass.)
//   L2 -> LDS    : every workgroup streams the same 64 KB (two operand stages of a 256 x 256 tile: L2 hits after the
//                  first pass) into LDS with direct-to-LDS loads, as the K loop's staging does, and nothing else.
//   L2 -> VGPR   : the same 64 KB per pass with 16-byte loads into registers (the other way to stage an operand).
//   LDS -> VGPR  : 16-byte LDS reads, conflict free, 8 KB per wavefront and pass (what the fragment reads can get).
//
// Each wavefront also reads the shader-clock counter and the 100 MHz counter at its start and end: their ratio is
// the clock the compute unit ran at under that load.
#include "../../include/dion_amd.h"
#include "common.h"
#include "mfma_tile.h"

namespace {

struct ProbeOut {
  unsigned long long t0, t1;   // 100 MHz counter
  unsigned long long c0, c1;   // shader clock counter
};

__global__ __launch_bounds__(512) void probe_mfma_kernel(const bf16_t* __restrict__ src, int iters, ProbeOut* out,
                                                         float* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // operands: 4 + 2 fragments of 8 bf16 per lane, from memory (so that they are not compile-time constants)
  bf16x8_t fa[4], fb[2];
  const u32x4_t* s = reinterpret_cast<const u32x4_t*>(src) + (size_t)((blockIdx.x * 8 + wave) * 64 + lane) * 6;
#pragma unroll
  for (int i = 0; i < 4; ++i) fa[i] = __builtin_bit_cast(bf16x8_t, s[i]);
#pragma unroll
  for (int j = 0; j < 2; ++j) fb[j] = __builtin_bit_cast(bf16x8_t, s[4 + j]);
  f32x16_t acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int rep = 0; rep < 4; ++rep)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memrealtime(), c1 = __builtin_amdgcn_s_memtime();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) r += acc[i][j][v];
  if (r == 12345.678f) sink[0] = r;   // keeps the accumulators alive
  if (lane == 0) out[blockIdx.x * 8 + wave] = ProbeOut{t0, t1, c0, c1};
}

// The same with v_mfma_f32_16x16x32_bf16 (half the flops per instruction, sixteen independent accumulators).
__global__ __launch_bounds__(512) void probe_mfma16_kernel(const bf16_t* __restrict__ src, int iters, ProbeOut* out,
                                                           float* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  bf16x8_t fa[4], fb[4];
  const u32x4_t* s = reinterpret_cast<const u32x4_t*>(src) + (size_t)((blockIdx.x * 8 + wave) * 64 + lane) * 6;
#pragma unroll
  for (int i = 0; i < 4; ++i) fa[i] = __builtin_bit_cast(bf16x8_t, s[i]);
#pragma unroll
  for (int j = 0; j < 4; ++j) fb[j] = __builtin_bit_cast(bf16x8_t, s[2 + j]);
  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int rep = 0; rep < 4; ++rep)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memrealtime(), c1 = __builtin_amdgcn_s_memtime();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) r += acc[i][j][v];
  if (r == 12345.678f) sink[0] = r;
  if (lane == 0) out[blockIdx.x * 8 + wave] = ProbeOut{t0, t1, c0, c1};
}

__global__ __launch_bounds__(512) void probe_lds_stream_kernel(const char* __restrict__ src, int iters, ProbeOut* out,
                                                               float* sink) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = wave_uniform((int)(threadIdx.x >> 6));
  // 64 KB per pass: 64 wave-instructions of 1 KB, eight per wavefront; every workgroup of an XCD reads the same
  // 64 KB (one region per 32 workgroups), so everything after the first pass is an L2 hit
  const char* base = src + (size_t)(blockIdx.x >> 5) * 65536;
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
    char* st = lds + (it & 1) * 65536;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      dma16(base, (unsigned)(((i * 8 + wave) * 64 + lane) * 16), lds_addr(st) + (i * 8 + wave) * 1024);
    dma_wait();
    __syncthreads();
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memrealtime(), c1 = __builtin_amdgcn_s_memtime();
  if (reinterpret_cast<float*>(lds)[threadIdx.x] == 12345.678f) sink[0] = 1.f;
  if (lane == 0) out[blockIdx.x * 8 + wave] = ProbeOut{t0, t1, c0, c1};
}

// The same 64 KB per pass into registers (16-byte loads, one per lane and wave-instruction), no LDS involved.
__global__ __launch_bounds__(512) void probe_reg_stream_kernel(const char* __restrict__ src, int iters, ProbeOut* out,
                                                               float* sink) {
  const int lane = threadIdx.x & 63;
  const int wave = wave_uniform((int)(threadIdx.x >> 6));
  const char* base = src + (size_t)(blockIdx.x >> 5) * 65536;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
    u32x4_t v[8];
    const char* b = base;
    asm volatile("" : "+s"(b));     // (opaque per pass: the loads stay inside the loop)
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = ldg16(b + ((i * 8 + wave) * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc ^= v[i];
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memrealtime(), c1 = __builtin_amdgcn_s_memtime();
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) sink[0] = 1.f;
  if (lane == 0) out[blockIdx.x * 8 + wave] = ProbeOut{t0, t1, c0, c1};
}

// LDS reads alone: every wavefront reads 16 bytes per lane, conflict free (consecutive lanes, consecutive addresses),
// eight reads in flight, from a 64 KB region.
__global__ __launch_bounds__(512) void probe_lds_read_kernel(int iters, ProbeOut* out, float* sink) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = wave_uniform((int)(threadIdx.x >> 6));
  for (int i = threadIdx.x; i < 65536 / 4; i += 512) reinterpret_cast<float*>(lds)[i] = (float)i;
  __syncthreads();
  u32x4_t acc = {0u, 0u, 0u, 0u};
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
    u32x4_t v[8];
    unsigned off = (unsigned)(it & 7) * 8192u;
    asm volatile("" : "+s"(off));   // (opaque per pass: the reads stay inside the loop)
    const char* b = lds + off;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const u32x4_t*>(b + ((i ^ wave) & 7) * 1024 + lane * 16);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc ^= v[i];
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memrealtime(), c1 = __builtin_amdgcn_s_memtime();
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) sink[0] = 1.f;
  if (lane == 0) out[blockIdx.x * 8 + wave] = ProbeOut{t0, t1, c0, c1};
}

}  // namespace

extern "C" int dion_amd_probe(int which, const void* random_src, size_t src_bytes, int iters, void* records,
                              size_t record_bytes, float* sink, double* ms, void* stream) {
  if (!random_src || !records || !sink || !ms || iters < 1) return DA_ERR_ARG;
  const int grid = da_cu_count();
  if (record_bytes < (size_t)grid * 8 * sizeof(ProbeOut)) return DA_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipEvent_t e0, e1;
  DA_HIP_CHECK(hipEventCreate(&e0));
  DA_HIP_CHECK(hipEventCreate(&e1));
  int rc = DA_OK;
  if (which == 0) {
    if (src_bytes < (size_t)grid * 8 * 64 * 6 * 16) return DA_ERR_WORKSPACE;
    DA_HIP_CHECK(hipEventRecord(e0, s));
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(grid), dim3(512), 0, s, static_cast<const bf16_t*>(random_src), iters,
                       static_cast<ProbeOut*>(records), sink);
    rc = da_launch_status();
  } else if (which == 1) {
    if (src_bytes < (size_t)((grid + 31) / 32) * 65536) return DA_ERR_WORKSPACE;
    static DaOncePerDevice configured;
    rc = configured.run([&]() -> int {
      DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(probe_lds_stream_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
      return DA_OK;
    });
    if (rc) return rc;
    DA_HIP_CHECK(hipEventRecord(e0, s));
    hipLaunchKernelGGL(probe_lds_stream_kernel, dim3(grid), dim3(512), 131072, s, static_cast<const char*>(random_src),
                       iters, static_cast<ProbeOut*>(records), sink);
    rc = da_launch_status();
  } else if (which == 2) {
    if (src_bytes < (size_t)((grid + 31) / 32) * 65536) return DA_ERR_WORKSPACE;
    DA_HIP_CHECK(hipEventRecord(e0, s));
    hipLaunchKernelGGL(probe_reg_stream_kernel, dim3(grid), dim3(512), 0, s, static_cast<const char*>(random_src), iters,
                       static_cast<ProbeOut*>(records), sink);
    rc = da_launch_status();
  } else if (which == 4) {
    if (src_bytes < (size_t)grid * 8 * 64 * 6 * 16) return DA_ERR_WORKSPACE;
    DA_HIP_CHECK(hipEventRecord(e0, s));
    hipLaunchKernelGGL(probe_mfma16_kernel, dim3(grid), dim3(512), 0, s, static_cast<const bf16_t*>(random_src), iters,
                       static_cast<ProbeOut*>(records), sink);
    rc = da_launch_status();
  } else if (which == 3) {
    static DaOncePerDevice configured;
    rc = configured.run([&]() -> int {
      DA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(probe_lds_read_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
      return DA_OK;
    });
    if (rc) return rc;
    DA_HIP_CHECK(hipEventRecord(e0, s));
    hipLaunchKernelGGL(probe_lds_read_kernel, dim3(grid), dim3(512), 65536, s, iters, static_cast<ProbeOut*>(records), sink);
    rc = da_launch_status();
  } else {
    return DA_ERR_ARG;
  }
  if (rc) return rc;
  DA_HIP_CHECK(hipEventRecord(e1, s));
  DA_HIP_CHECK(hipEventSynchronize(e1));
  float t = 0.f;
  DA_HIP_CHECK(hipEventElapsedTime(&t, e0, e1));
  *ms = t;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return DA_OK;
}
