// Measurement probe: what the matrix pipes of this GPU sustain on nothing but bf16 MFMAs, as a function of how much
// the operands change from one instruction to the next.  Under a power or current limit the clock, and with it the
// rate, depends on that activity; the attention and GEMM kernels are judged against the rate measured here next to
// the published peak.  Not part of the drop-in boundary and not part of libringattn_hip.so: it is built into
// libringattn_probe.so, which only the benchmark and its test load (declared in ringattn_hip_measure.h).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../../include/ringattn_hip_measure.h"

namespace ra {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// MODE 0: one value in every lane and register; 1: a value per lane and register, the same in every instruction;
// 2: random values, and consecutive instructions of an accumulator see different operand pairs (eight A and eight B
// registers, all 64 pairings in turn)
template <int MODE>
__global__ __launch_bounds__(256) void mfma_probe_kernel(float* sink, int iters) {
  bf16x8 a[8], b[8];
  uint32_t s = threadIdx.x * 2654435761u + 12345u;
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      float x = 0.5f, y = 0.25f;
      if (MODE == 1) { x = threadIdx.x * 0.001f + e; y = threadIdx.x * 0.002f - e; }
      if (MODE == 2) {
        s = s * 1664525u + 1013904223u; x = ((int)(s >> 8) - (1 << 23)) * (1.f / (1 << 23));
        s = s * 1664525u + 1013904223u; y = ((int)(s >> 8) - (1 << 23)) * (1.f / (1 << 23));
      }
      a[i][e] = (__bf16)x; b[i][e] = (__bf16)y;
    }
  f32x16 c[4];
#pragma unroll
  for (int m = 0; m < 4; m++)
#pragma unroll
    for (int r = 0; r < 16; r++) c[m][r] = 0.f;
  for (int it = 0; it < iters; it++) {      // 64 MFMAs per iteration, four independent accumulators
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
      for (int i = 0; i < 8; i++)
        c[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[MODE == 2 ? (i + j) & 7 : i], c[i & 3], 0, 0, 0);
  }
  float t = 0.f;
#pragma unroll
  for (int m = 0; m < 4; m++)
#pragma unroll
    for (int r = 0; r < 16; r++) t += c[m][r];
  sink[blockIdx.x * 256 + threadIdx.x] = t;
}

}  // namespace ra

extern "C" int ra_mfma_rate_probe(float* sink, int32_t workgroups, int32_t iters, int32_t operands, ra_stream_t stream) {
  if (!sink || workgroups <= 0 || workgroups > 65536 || iters <= 0 || iters > (1 << 22) || operands < 0 || operands > 2)
    return RA_ERR_INVALID;
  hipStream_t s = (hipStream_t)stream;
  if (operands == 0) ra::mfma_probe_kernel<0><<<workgroups, 256, 0, s>>>(sink, iters);
  else if (operands == 1) ra::mfma_probe_kernel<1><<<workgroups, 256, 0, s>>>(sink, iters);
  else ra::mfma_probe_kernel<2><<<workgroups, 256, 0, s>>>(sink, iters);
  return hipGetLastError() == hipSuccess ? RA_OK : RA_ERR_LAUNCH;
}
