// Measurement aid: what the matrix cores sustain when nothing else runs.  One wave per SIMD issues
// independent 32x32x16 bf16 MFMAs back to back on operands it holds in registers (no LDS, no
// memory traffic inside the timed part) and reports the shader cycles and the 100 MHz real-time
// ticks it took, so that the clock the chip holds under that load can be read off.  With operands
// of zeros the chip stays at its full clock; with N(0,1)-like operands the power cap lowers the
// clock, which is the ceiling that the GEMM kernels of this library work under on real data.
// Not part of libflashmuon_hip.so: built into libflashmuon_probe.so, which only bench.py --mfma-probe loads.
#include "../fm_internal.h"

namespace fm {
namespace {

__global__ __launch_bounds__(256) void mfma_peak_kernel(const uint4* __restrict__ src, float* sink, long long* clocks, int iters) {
  const int tid = threadIdx.x;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint4 u = src[(blockIdx.x * 256 + tid) * 8 + i], v = src[(blockIdx.x * 256 + tid) * 8 + 4 + i];
    a[i] = __builtin_bit_cast(bf16x8_t, u);
    b[i] = __builtin_bit_cast(bf16x8_t, v);
  }
  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const long long c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
  for (int it = 0; it < iters; ++it)
#pragma unroll
    for (int q = 0; q < 64; ++q)   // 4 k16 substeps of a 128 x 128 block: 64 MFMAs, as one k stage of the GEMM
      acc[(q >> 2) & 3][q & 3] = mfma_32x32x16<false>(a[(q >> 2) & 3], b[q & 3], acc[(q >> 2) & 3][q & 3]);
  const long long c1 = __builtin_readcyclecounter(), r1 = wall_clock64();
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  sink[blockIdx.x * 256 + tid] = s;
  if (tid == 0) {
    clocks[blockIdx.x * 2] = c1 - c0;
    clocks[blockIdx.x * 2 + 1] = r1 - r0;
  }
}

}  // namespace
}  // namespace fm

// `launches` launches of a kernel in which `blocks` workgroups of four waves each issue iters * 64
// independent 32x32x16 bf16 MFMAs per wave on register operands taken from `operands` (blocks * 256 *
// 128 bytes: zeros, or N(0,1) bf16 values).  After the last launch clocks[2*b] holds the shader cycles
// and clocks[2*b + 1] the 100 MHz real-time ticks workgroup b spent in its loop; sink takes
// blocks * 256 floats nobody needs.  The flop count is blocks * 4 * iters * 64 * 32768 per launch.
// Returns 0, or 1 (a NULL pointer), 2 (a count out of range), 7 (launch failed).
extern "C" __attribute__((visibility("default")))
int fm_probe_mfma_peak(const void* operands, int blocks, int iters, int launches, float* sink,
                       long long* clocks, void* stream) {
  if (!operands || !sink || !clocks) return 1;
  if (blocks <= 0 || blocks > 1024 || iters <= 0 || launches <= 0) return 2;
  for (int i = 0; i < launches; ++i)
    hipLaunchKernelGGL(fm::mfma_peak_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(operands), sink, clocks, iters);
  return hipGetLastError() == hipSuccess ? 0 : 7;
}
