// Bench-only measurement kernels (no counterpart in the reference and no part of the product
// library): built into libflexprobe.so, which only bench.py and a GPU test load.
//   flexprobe_mfma   nothing but v_mfma_f32_32x32x16_f16 on pseudo-random operands
//   flexprobe_mix    the instruction mix of a fused attention step
//   flexprobe_read   a bare streaming read
// Each returns 0 on success; flexprobe_last_error() gives the message otherwise.
//
// Measurement aid (no counterpart in the reference): a kernel that does nothing but
// v_mfma_f32_32x32x16_f16 on pseudo-random operands, two waves per SIMD, four independent
// accumulators per wave.  Timing it gives the matrix throughput this GPU sustains under its
// power limit, which is what the fused kernels' TFLOP/s should be read against next to the
// published peak.
#include "mfma_common.cuh"

namespace flex {

__global__ __launch_bounds__(256, 2) void mfma_probe_kernel(float* __restrict__ sink, int iters) {
  float16_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[j][i] = 0.f;
  half8_t a[4], b[4];
  unsigned x = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
  for (int s = 0; s < 4; s++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      x = x * 1664525u + 1013904223u;
      a[s][e] = (_Float16)((float)((x >> 9) & 2047) * (1.f / 1024.f) - 1.f);
      x = x * 1664525u + 1013904223u;
      b[s][e] = (_Float16)((float)((x >> 9) & 2047) * (1.f / 1024.f) - 1.f);
    }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int m = 0; m < 8; m++) acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m & 3], b[(m >> 1) & 3], acc[m & 3], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[j][i];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

// Second aid: the instruction mix of a fused attention step.  Per "unit" a wave issues NM
// matrix instructions interleaved with 80 fused multiply-adds and 16 exponentials on 16
// registers (what scaling, score_mod, exp, rounding and row sums cost per 32x32 score block),
// two waves per SIMD.  NM = 8 is the forward at D = 64, 12 the dQ kernel, 16 the dK/dV kernel
// or the forward at D = 128.  Its rate is the ceiling of that mix on this GPU: matrix and
// vector instructions share the issue port and the power budget.
template <int NM>
__global__ __launch_bounds__(256, 2) void mix_probe_kernel(float* __restrict__ sink, int iters, float c0, float c1) {
  float16_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[j][i] = 0.f;
  half8_t a[4], b[4];
  unsigned x = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
  for (int s = 0; s < 4; s++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      x = x * 1664525u + 1013904223u;
      a[s][e] = (_Float16)((float)((x >> 9) & 2047) * (1.f / 1024.f) - 1.f);
      x = x * 1664525u + 1013904223u;
      b[s][e] = (_Float16)((float)((x >> 9) & 2047) * (1.f / 1024.f) - 1.f);
    }
  float y[16];
#pragma unroll
  for (int r = 0; r < 16; r++) y[r] = (float)a[r & 3][r >> 2];
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int m = 0; m < NM; m++) acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m & 3], b[(m >> 2) & 3], acc[m & 3], 0, 0, 0);
#pragma unroll
    for (int j = 0; j < 5; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) y[r] = __builtin_fmaf(y[r], c0, c1);
#pragma unroll
    for (int r = 0; r < 16; r++) y[r] = fast_exp2(y[r]);
#pragma unroll
    for (int m = 0; m < NM; m++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 80 / NM, 0);
      __builtin_amdgcn_sched_group_barrier(0x400, 16 / NM, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[j][i];
#pragma unroll
  for (int r = 0; r < 16; r++) s += y[r];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace flex

#include <cstdarg>
#include <cstdio>
static thread_local char g_probe_err[256] = "";
static void flex_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_probe_err, sizeof(g_probe_err), fmt, ap);
  va_end(ap);
}
extern "C" const char* flexprobe_last_error(void) { return g_probe_err; }

namespace flex {
// A streaming read and nothing else: every thread folds NLD independent 16-byte loads per trip into a value that
// is practically never written.  Consecutive threads read consecutive 16-byte pieces; a workgroup walks the buffer
// in strides of the whole grid, so at any time the grid covers one contiguous window.
template <int NLD>
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ src, size_t n_vec, float* __restrict__ sink) {
  const size_t tid = blockIdx.x * (size_t)blockDim.x + threadIdx.x, total = (size_t)gridDim.x * blockDim.x;
  uint4 acc = make_uint4(0, 0, 0, 0);
  for (size_t i = tid; i < n_vec; i += NLD * total) {
    uint4 x[NLD];
#pragma unroll
    for (int j = 0; j < NLD; j++) x[j] = i + j * total < n_vec ? src[i + j * total] : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < NLD; j++) { acc.x ^= x[j].x; acc.y ^= x[j].y; acc.z ^= x[j].z; acc.w ^= x[j].w; }
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[tid & 0xffff] = 1.f;
}
}  // namespace flex

// `workgroups` x 256 threads over `bytes` of device memory, `loads_in_flight` (1, 2, 4, 8 or 16) independent 16-byte
// loads per thread and trip.  workgroups <= 0: 1024; loads_in_flight <= 0: 4.  `sink`: 65536 floats.
extern "C" int flexprobe_read(const void* src, size_t bytes, float* sink, int32_t workgroups, int32_t loads_in_flight, void* stream) {
  if (!src || !sink || bytes < 16 || ((uintptr_t)src & 15)) {
    flex_set_error("flexprobe_read: needs a 16-byte aligned device buffer of at least 16 bytes and a sink of 65536 floats");
    return 1;
  }
  if (workgroups <= 0) workgroups = 1024;
  if (loads_in_flight <= 0) loads_in_flight = 4;
  const dim3 grid(workgroups), block(256);
  hipStream_t st = (hipStream_t)stream;
  const uint4* s4 = (const uint4*)src;
  const size_t n = bytes / 16;
  switch (loads_in_flight) {
    case 1: hipLaunchKernelGGL(flex::read_probe_kernel<1>, grid, block, 0, st, s4, n, sink); break;
    case 2: hipLaunchKernelGGL(flex::read_probe_kernel<2>, grid, block, 0, st, s4, n, sink); break;
    case 4: hipLaunchKernelGGL(flex::read_probe_kernel<4>, grid, block, 0, st, s4, n, sink); break;
    case 8: hipLaunchKernelGGL(flex::read_probe_kernel<8>, grid, block, 0, st, s4, n, sink); break;
    case 16: hipLaunchKernelGGL(flex::read_probe_kernel<16>, grid, block, 0, st, s4, n, sink); break;
    default: flex_set_error("flexprobe_read: loads_in_flight must be 1, 2, 4, 8 or 16"); return 1;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { flex_set_error("flexprobe_read: launch failed: %s", hipGetErrorString(e)); return 2; }
  return 0;
}

// 512 workgroups of 4 waves (two waves per SIMD on 256 compute units), 8 * iters MFMAs per wave.
extern "C" int flexprobe_mfma(float* sink, int32_t iters, double* flops_per_launch, void* stream) {
  if (!sink || iters <= 0) { flex_set_error("flexprobe_mfma: needs a device buffer of 512*256 floats and iters > 0"); return 1; }
  hipLaunchKernelGGL(flex::mfma_probe_kernel, dim3(512), dim3(256), 0, (hipStream_t)stream, sink, iters);
  if (flops_per_launch) *flops_per_launch = 512.0 * 4 * 8.0 * iters * 2.0 * 32 * 32 * 16;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { flex_set_error("flexprobe_mfma: launch failed: %s", hipGetErrorString(e)); return 2; }
  return 0;
}

// Same grid; `iters` units of `mfma_per_unit` (8, 12 or 16) matrix instructions + 96 vector instructions per wave.
extern "C" int flexprobe_mix(float* sink, int32_t iters, int32_t mfma_per_unit, double* flops_per_launch, void* stream) {
  if (!sink || iters <= 0 || (mfma_per_unit != 8 && mfma_per_unit != 12 && mfma_per_unit != 16)) {
    flex_set_error("flexprobe_mix: needs a device buffer of 512*256 floats, iters > 0 and mfma_per_unit in {8, 12, 16}");
    return 1;
  }
  hipStream_t st = (hipStream_t)stream;
  if (mfma_per_unit == 8) hipLaunchKernelGGL(flex::mix_probe_kernel<8>, dim3(512), dim3(256), 0, st, sink, iters, 0.999f, 0.001f);
  else if (mfma_per_unit == 12) hipLaunchKernelGGL(flex::mix_probe_kernel<12>, dim3(512), dim3(256), 0, st, sink, iters, 0.999f, 0.001f);
  else hipLaunchKernelGGL(flex::mix_probe_kernel<16>, dim3(512), dim3(256), 0, st, sink, iters, 0.999f, 0.001f);
  if (flops_per_launch) *flops_per_launch = 512.0 * 4 * (double)mfma_per_unit * iters * 2.0 * 32 * 32 * 16;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { flex_set_error("flexprobe_mix: launch failed: %s", hipGetErrorString(e)); return 2; }
  return 0;
}
