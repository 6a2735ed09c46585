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

// SHAPE 0: 64 MFMAs 32x32x16 per iteration (a 128x128 block over one 64-wide k stage, as in the GEMM);
// SHAPE 1: the same flops as 128 MFMAs 16x16x32 (8 x 8 accumulator tiles, two k32 steps).
// LDS: every 16 (SHAPE 0) or 32 (SHAPE 1) MFMAs are accompanied by eight 16-byte LDS reads per lane, the
// fragment traffic of the GEMM's main loop; what is read replaces the operands.
template <int SHAPE, bool LDS>
__global__ __launch_bounds__(256) void mfma_peak_kernel(const uint4* __restrict__ src, float* sink, long long* clocks, int iters) {
  __shared__ uint4 lds[LDS ? 8 * 256 : 1];
  const int tid = threadIdx.x;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint4 u = src[(blockIdx.x * 256 + tid) * 8 + i], v = src[(blockIdx.x * 256 + tid) * 8 + 4 + i];
    a[i] = __builtin_bit_cast(bf16x8_t, u);
    b[i] = __builtin_bit_cast(bf16x8_t, v);
    if (LDS) { lds[i * 256 + tid] = u; lds[(4 + i) * 256 + tid] = v; }
  }
  if (LDS) __syncthreads();
  float s = 0.0f;
  long long c0, c1, r0, r1;
  if constexpr (SHAPE == 0) {
    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    c0 = __builtin_readcyclecounter(); r0 = wall_clock64();
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int q = 0; q < 64; ++q) {
        if (LDS && (q & 15) < 8) {   // conflict free: lane l reads 16 bytes at 16 l of a 4 KiB row
          const uint4 u = lds[(q & 7) * 256 + ((tid + 64 * (q >> 4)) & 255)];
          if ((q & 7) < 4) a[q & 3] = __builtin_bit_cast(bf16x8_t, u); else b[q & 3] = __builtin_bit_cast(bf16x8_t, u);
        }
        acc[(q >> 2) & 3][q & 3] = mfma_32x32x16<false>(a[(q >> 2) & 3], b[q & 3], acc[(q >> 2) & 3][q & 3]);
      }
    c1 = __builtin_readcyclecounter(); r1 = wall_clock64();
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  } else {
    f32x4_t acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
    c0 = __builtin_readcyclecounter(); r0 = wall_clock64();
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int q = 0; q < 128; ++q) {
        if (LDS && (q & 31) < 8) {
          const uint4 u = lds[(q & 7) * 256 + ((tid + 64 * (q >> 5)) & 255)];
          if ((q & 7) < 4) a[q & 3] = __builtin_bit_cast(bf16x8_t, u); else b[q & 3] = __builtin_bit_cast(bf16x8_t, u);
        }
        const int i = (q >> 3) & 7, j = q & 7;
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 3], b[j & 3], acc[i][j], 0, 0, 0);
      }
    c1 = __builtin_readcyclecounter(); r1 = wall_clock64();
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) s += acc[i][j][r];
  }
  sink[blockIdx.x * 256 + tid] = s;
  if (tid == 0) {
    clocks[blockIdx.x * 2] = c1 - c0;
    clocks[blockIdx.x * 2 + 1] = r1 - r0;
  }
}

}  // namespace
}  // namespace fm

// `launches` launches of a kernel in which `blocks` workgroups of four waves each issue, per wave and
// iteration, 64 independent 32x32x16 bf16 MFMAs (shape 0) or the same flops as 128 MFMAs 16x16x32
// (shape 1), on register operands taken from `operands` (blocks * 256 * 128 bytes: zeros, or N(0,1)
// bf16 values); with lds != 0 the loop also reads fragments from LDS at the rate of the GEMM's main
// loop.  After the last launch clocks[2*b] holds the shader cycles and clocks[2*b + 1] the 100 MHz
// real-time ticks workgroup b spent in its loop; sink takes blocks * 256 floats nobody needs.  The
// flop count is blocks * 4 * iters * 64 * 32768 per launch.
// Returns 0, or 1 (a NULL pointer), 2 (a count out of range), 7 (launch failed).
extern "C" __attribute__((visibility("default")))
int fm_probe_mfma_peak(const void* operands, int blocks, int iters, int launches, float* sink,
                       long long* clocks, void* stream, int shape, int lds) {
  if (!operands || !sink || !clocks) return 1;
  if (blocks <= 0 || blocks > 1024 || iters <= 0 || launches <= 0 || shape < 0 || shape > 1) return 2;
  for (int i = 0; i < launches; ++i) {
#define FM_PROBE(S, L) hipLaunchKernelGGL((fm::mfma_peak_kernel<S, L>), dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), \
                                          static_cast<const uint4*>(operands), sink, clocks, iters)
    if (shape == 0) { if (lds) FM_PROBE(0, true); else FM_PROBE(0, false); }
    else { if (lds) FM_PROBE(1, true); else FM_PROBE(1, false); }
#undef FM_PROBE
  }
  return hipGetLastError() == hipSuccess ? 0 : 7;
}
