// A measuring stick, not part of any convolution: the rate at which the chip retires
// v_mfma_i32_32x32x32_i8 when nothing else is in the way (operands in registers, eight independent
// accumulator tiles per wave, no memory traffic inside the loop).  The roofline fractions of the MFMA
// kernels are quoted against the published peak; this probe says what the instruction itself reaches.
// Built into a library of its own (libehip_probe.so) that only the benchmark loads: it is no interface of
// the convolution path and the product library does not export it.
//
//   ehip_bench_probe_mfma_i8: launches `workgroups` x 4 waves that each retire 8 x iters MFMAs from
//   registers and writes one int per thread (workgroups x 256) to out_dev; *ops_out = the integer
//   operations issued.  The caller times it.
#include "ehip_internal.hpp"

namespace ehip {

__global__ __launch_bounds__(kBlock) void k_probe_mfma_i8(int iters, int *out)
{
  v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {(int)blockIdx.x, 5, 6, 7};
  v16i acc[8];
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[t], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[t][v];
  out[(size_t)blockIdx.x * kBlock + threadIdx.x] = s;
}

}  // namespace ehip

using namespace ehip;

extern "C" __attribute__((visibility("default"))) int ehip_bench_probe_mfma_i8(int workgroups, int iters, void *out_dev, double *ops_out, void *hip_stream)
{
  if (workgroups < 1 || workgroups > 65536 || iters < 1 || !out_dev) return EHIP_GENERAL_ERROR;
  hipLaunchKernelGGL(k_probe_mfma_i8, dim3(workgroups), dim3(kBlock), 0, static_cast<hipStream_t>(hip_stream), iters,
                     static_cast<int *>(out_dev));
  if (ops_out) *ops_out = (double)workgroups * (kBlock / 64) * (double)iters * 8.0 * 2.0 * 32 * 32 * 32;
  return hipGetLastError() == hipSuccess ? EHIP_OK : EHIP_GENERAL_ERROR;
}
