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

}  // namespace flex

void flex_set_error(const char* fmt, ...);

// 512 workgroups of 4 waves (two waves per SIMD on 256 compute units), 8 * iters MFMAs per wave.
extern "C" int flexattn_probe_mfma(float* sink, int32_t iters, double* flops_per_launch, void* stream) {
  if (!sink || iters <= 0) { flex_set_error("flexattn_probe_mfma: needs a device buffer of 512*256 floats and iters > 0"); return 1; }
  hipLaunchKernelGGL(flex::mfma_probe_kernel, dim3(512), dim3(256), 0, (hipStream_t)stream, sink, iters);
  if (flops_per_launch) *flops_per_launch = 512.0 * 4 * 8.0 * iters * 2.0 * 32 * 32 * 16;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { flex_set_error("flexattn_probe_mfma: launch failed: %s", hipGetErrorString(e)); return 2; }
  return 0;
}
