// Measurement aid: the rate at which the matrix pipe runs the scaled MFMA instruction out of registers alone
// (no LDS, no memory traffic), as a function of the operand bits.  The GEMM kernels' roofline is quoted against the
// chip's nominal peak; this loop shows what the chip sustains on a given kind of data when nothing but the matrix
// pipe works, which is the ceiling any schedule of the same instructions has on that data.
#include "mx_common.h"

namespace mx {
namespace {

// Every wave keeps 8 A fragments and 4 B fragments (the register tile of the ping-pong GEMM kernel) and multiplies
// all 32 pairs `iters` times; two waves per SIMD, as in that kernel.  `frags`: 12 x 512 fragments of 32 bytes
// ([fragment][thread]); FP4 uses the first 16 bytes of each.
template <int FMT>
__global__ __launch_bounds__(512) void mfma_rate_kernel(const v8i* __restrict__ frags, float* __restrict__ sink,
                                                        int iters) {
  v8i a[8], b[4];
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = frags[i * 512 + t];
#pragma unroll
  for (int j = 0; j < 4; ++j) b[j] = frags[(8 + j) * 512 + t];
  v4f acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  const int one = 0x7F7F7F7F;   // scale bytes 127 = 1.0
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[j], a[i], acc[i][j], FMT, FMT, 0, one, 0, one);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s += acc[i][j].x + acc[i][j].y + acc[i][j].z + acc[i][j].w;
  sink[blockIdx.x * 512 + t] = s;
}

}  // namespace
}  // namespace mx

extern "C" int mx_probe_mfma_rate(int32_t fmt, const void* frags, int32_t workgroups, int32_t iters, float* sink,
                                  void* stream) {
  using namespace mx;
  if (!frags || !sink || workgroups <= 0 || iters <= 0)
    return set_error(MX_ERR_INVALID, "mx_probe_mfma_rate: null pointer or non-positive size");
  if (((uintptr_t)frags) % 32 != 0) return set_error(MX_ERR_LAYOUT, "mx_probe_mfma_rate: frags must be 32-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (fmt == MX_E4M3)
    hipLaunchKernelGGL(mfma_rate_kernel<MX_E4M3>, dim3(workgroups), dim3(512), 0, st, (const v8i*)frags, sink,
                       iters);
  else if (fmt == MX_E5M2)
    hipLaunchKernelGGL(mfma_rate_kernel<MX_E5M2>, dim3(workgroups), dim3(512), 0, st, (const v8i*)frags, sink,
                       iters);
  else if (fmt == MX_E2M1)
    hipLaunchKernelGGL(mfma_rate_kernel<MX_E2M1>, dim3(workgroups), dim3(512), 0, st, (const v8i*)frags, sink,
                       iters);
  else
    return set_error(MX_ERR_DTYPE, "mx_probe_mfma_rate: fmt must be MX_E4M3, MX_E5M2 or MX_E2M1");
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "mfma_rate_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}
