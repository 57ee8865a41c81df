// Matrix-pipe rate probe: a loop of independent v_mfma_f32_32x32x16_bf16 on register operands, eight
// waves per workgroup, one workgroup per compute unit.  The sustained MFMA rate of this GPU is set
// by its power limit and depends on the operand bits (zeros run near the nominal clock, random
// operands several hundred MHz lower), so a roofline fraction against the nominal peak says little
// without this number measured next to it on the same device with the same kind of data.
//
// Built into bench_probe.so beside bench.py, which is its only user; it is not part of libmoda_hip.so.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "moda_amd/csrc/tile.h"

namespace moda {

__global__ __launch_bounds__(512) void mfma_probe_kernel(const i32x4* operands, int64_t iters, uint64_t* clocks,
                                                         float* sink) {
  const int lane = threadIdx.x & 63;
  i32x4 a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    a[j] = operands[j * 64 + lane];
    b[j] = operands[256 + j * 64 + lane];
  }
  f32x16 c[4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) c[i][j] = 0.f;
  const uint64_t t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int64_t it = 0; it < iters; it++) {
#pragma unroll
    for (int q = 0; q < 4; q++) c[q] = mfma32<BF16>(a[q], b[q], c[q]);
  }
  const uint64_t t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (clocks && blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = t1 - t0;  // shader-clock cycles spent in the loop
    clocks[1] = r1 - r0;  // the same interval on the constant 100 MHz counter
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++) s += c[i][i];
  if (s == 12345.678f) sink[0] = s;  // keeps the loop alive; practically never true
}

}  // namespace moda

// Runs `iters` rounds of four independent bf16 MFMAs per wave (eight waves per workgroup, `workgroups`
// workgroups; 32768 FLOP per MFMA) on the register operands found in `operands` (device memory, 512 x 16
// bytes: lane l of operand j reads entry 64*j + l; entries 0..255 feed the A side, 256..511 the B side).
// `clocks` (device, two uint64, may be NULL) receives the loop's duration in shader-clock cycles and in
// 100 MHz ticks; `sink` is 4 bytes of device scratch.  Returns 0, -1 for bad arguments, -2 for a failed launch.
extern "C" int bench_probe_mfma(const void* operands, int64_t iters, int64_t workgroups, uint64_t* clocks, float* sink,
                                void* stream) {
  if (!operands || !sink || iters < 0 || workgroups <= 0 || workgroups > (1 << 20)) return -1;
  if ((uintptr_t)operands % 16 != 0) return -1;
  hipLaunchKernelGGL(moda::mfma_probe_kernel, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream,
                     reinterpret_cast<const moda::i32x4*>(operands), iters, clocks, sink);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
