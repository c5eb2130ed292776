// Skinny-M ("decode") block-scaled GEMM: C[M<=32, N] = X[M, K] (8-bit MX) x W[N, K] (MXFP4) ^T.
//
// The problem is bound by streaming W (and its scales) from HBM exactly once, so the kernel is
// organised around keeping many bytes in flight rather than around tile reuse:
//   * a workgroup of 8 waves owns a run of 16-row tiles of W; wave w owns K-slice w (SPW MFMA K-steps
//     of 128 elements) of every tile, so the 8 waves together read each tile's rows contiguously;
//   * each wave keeps its K-slice of X resident in VGPRs for the whole kernel (X is tiny and shared
//     by all workgroups through L2), so W is the only stream;
//   * W fragments go global -> VGPR directly in MFMA operand layout (4-bit: lane (r, g) holds row r and
//     the 32-element block g of a K-step, so the four lane groups read 64 contiguous bytes of a row;
//     8-bit X: bytes 16 g .. and 64 + 16 g .. of the K-step), the next tile's loads are issued before
//     the current tile's MFMAs;
//   * v_mfma_scale_f32_16x16x128_f8f6f4 with mixed formats (W as FP4 first matrix, X as FP8 second
//     matrix), E8M0 scales read in place from the [N, K/32] / [M, K/32] tensors;
//   * the 8 K-slice partial sums meet in LDS and 128 threads write the bf16/fp32 result.
#include "mx_common.h"

namespace mx {
namespace {

constexpr int kWaves = 8;

template <int XF, int SPW, int MT, typename OutT>
__global__ __launch_bounds__(kWaves * 64) void decode_kernel(const DecodeArgs d) {
  __shared__ v4f red[2][kWaves][MT][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, gq = lane >> 4;
  const int ksteps = d.K / 128;
  const int s0 = wave * SPW;   // first K-step of this wave's slice

  // ---- resident X fragments and scales ---------------------------------------------------------------
  v8i xf[MT][SPW];
  int xs[MT][(SPW + 3) / 4];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = 16 * i + r;
    const bool mok = m < d.M;
#pragma unroll
    for (int u = 0; u < (SPW + 3) / 4; ++u) xs[i][u] = 0x7F7F7F7F;
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      v8i f = {0, 0, 0, 0, 0, 0, 0, 0};
      int sc = 127;
      if (mok && s0 + s < ksteps) {
        // 8-bit operand layout of the MFMA: bytes 16 g .. 16 g + 15 and 64 + 16 g .. of the K-step
        const uint8_t* p = d.X + (int64_t)m * d.ldx + (int64_t)(s0 + s) * 128 + gq * 16;
        const v4i lo = *(const v4i*)p, hi = *(const v4i*)(p + 64);
        f = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        sc = d.Xs[(int64_t)m * d.ldxs + (s0 + s) * 4 + gq];
      }
      xf[i][s] = f;
      xs[i][s / 4] = (xs[i][s / 4] & ~(0xFF << (8 * (s % 4)))) | (sc << (8 * (s % 4)));
    }
  }

  const int tiles = d.N / 16;
  // contiguous run of tiles per workgroup
  const int per = tiles / gridDim.x, rem = tiles % gridDim.x;
  const int b = blockIdx.x;
  const int t_begin = b * per + (b < rem ? b : rem);
  const int t_end = t_begin + per + (b < rem ? 1 : 0);

  // this lane's byte offsets inside a W row / scale row for its K-slice
  const int64_t wcol = (int64_t)s0 * 64 + gq * 16;   // FP4: 64 bytes per K-step, 16 per block
  const int64_t scol = (int64_t)s0 * 4;
  const bool slice_live = s0 < ksteps;

  v4i wb0[SPW], wb1[SPW];
  v4i ws0[(SPW + 3) / 4], ws1[(SPW + 3) / 4];

  auto load_tile = [&](int t, v4i* wb, v4i* wsc) {
    const uint8_t* wrow = d.W + (int64_t)(t * 16 + r) * d.ldw + wcol;
    const uint8_t* srow = d.Ws + (int64_t)(t * 16 + r) * d.ldws + scol;
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      if (s0 + s < ksteps) wb[s] = __builtin_nontemporal_load((const v4i*)(wrow + s * 64));
      else wb[s] = (v4i){0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < (SPW + 3) / 4; ++u) {
      // 16 scale bytes = K-steps 4u .. 4u+3 of the slice (4 blocks each)
      if (s0 + 4 * u < ksteps) wsc[u] = *(const v4i*)(srow + u * 16);
      else wsc[u] = (v4i){0x7F7F7F7F, 0x7F7F7F7F, 0x7F7F7F7F, 0x7F7F7F7F};
    }
  };

  auto compute_tile = [&](int t, int it, const v4i* wb, const v4i* wsc) {
    v4f acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    if (slice_live) {
#pragma unroll
      for (int s = 0; s < SPW; ++s) {
        const v8i wf = {wb[s].x, wb[s].y, wb[s].z, wb[s].w, 0, 0, 0, 0};
        // byte gq of dword s%4 of the scale vector u = s/4: the scale of block 4*(s0+s) + gq
        const int wscale = (int)((uint32_t)wsc[s / 4][s % 4] >> (8 * gq));
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          if (s % 4 == 0)
            acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[i][s], acc[i], MX_E2M1, XF, 0, wscale, 0, xs[i][s / 4]);
          else if (s % 4 == 1)
            acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[i][s], acc[i], MX_E2M1, XF, 0, wscale, 1, xs[i][s / 4]);
          else if (s % 4 == 2)
            acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[i][s], acc[i], MX_E2M1, XF, 0, wscale, 2, xs[i][s / 4]);
          else
            acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[i][s], acc[i], MX_E2M1, XF, 0, wscale, 3, xs[i][s / 4]);
        }
      }
    }
    const int rb = it & 1;
#pragma unroll
    for (int i = 0; i < MT; ++i) red[rb][wave][i][lane] = acc[i];
    __syncthreads();
    if (tid < MT * 64) {
      const int i = tid >> 6, l = tid & 63;
      v4f sum = red[rb][0][i][l];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) sum += red[rb][w][i][l];
      const int m = 16 * i + (l & 15);
      const int n = t * 16 + 4 * (l >> 4);
      if (m < d.M) {
        OutT* c = (OutT*)d.C + (int64_t)m * d.ldc + n;
        if constexpr (sizeof(OutT) == 4) {
          for (int e = 0; e < 4; ++e) c[e] = d.accumulate ? c[e] + sum[e] : sum[e];
        } else {
          for (int e = 0; e < 4; ++e)
            c[e] = f32_to_bf16(d.accumulate ? bf16_to_f32(c[e]) + sum[e] : sum[e]);
        }
      }
    }
  };

  if (t_begin >= t_end) return;   // uniform per workgroup
  load_tile(t_begin, wb0, ws0);
  int it = 0;
  for (int t = t_begin; t < t_end; t += 2) {
    if (t + 1 < t_end) load_tile(t + 1, wb1, ws1);
    compute_tile(t, it++, wb0, ws0);
    if (t + 1 < t_end) {
      if (t + 2 < t_end) load_tile(t + 2, wb0, ws0);
      compute_tile(t + 1, it++, wb1, ws1);
    }
  }
}

template <int XF, int SPW, int MT>
int launch_decode_t(const DecodeArgs& d, int grid, hipStream_t stream) {
  if (d.c_dtype == MX_F32)
    hipLaunchKernelGGL((decode_kernel<XF, SPW, MT, float>), dim3(grid), dim3(kWaves * 64), 0, stream, d);
  else
    hipLaunchKernelGGL((decode_kernel<XF, SPW, MT, uint16_t>), dim3(grid), dim3(kWaves * 64), 0, stream, d);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "decode_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

template <int XF>
int launch_decode_x(const DecodeArgs& d, int grid, hipStream_t stream) {
  const int ksteps = d.K / 128;
  const bool one = d.M <= 16;
  if (ksteps <= kWaves * 4)
    return one ? launch_decode_t<XF, 4, 1>(d, grid, stream) : launch_decode_t<XF, 4, 2>(d, grid, stream);
  return one ? launch_decode_t<XF, 8, 1>(d, grid, stream) : launch_decode_t<XF, 8, 2>(d, grid, stream);
}

}  // namespace

int launch_gemm_decode(const DecodeArgs& d, hipStream_t stream) {
  if (d.w_fmt != MX_E2M1) return set_error(MX_ERR_DTYPE, "decode kernel: weights must be MX_E2M1");
  if (d.x_fmt != MX_E4M3 && d.x_fmt != MX_E5M2) return set_error(MX_ERR_DTYPE, "decode kernel: activations must be 8-bit");
  if (d.M < 1 || d.M > 32) return set_error(MX_ERR_SHAPE, "decode kernel: M must be in 1..32");
  if (d.K % 512 != 0 || d.K > kWaves * 8 * 128)
    return set_error(MX_ERR_SHAPE, "decode kernel: K must be a multiple of 512 and at most %d", kWaves * 8 * 128);
  if (d.N % 16 != 0) return set_error(MX_ERR_SHAPE, "decode kernel: N must be a multiple of 16");
  if (((uintptr_t)d.X | (uintptr_t)d.W | (uintptr_t)d.Ws | (uintptr_t)d.ldx | (uintptr_t)d.ldw | (uintptr_t)d.ldws) % 16 != 0)
    return set_error(MX_ERR_LAYOUT, "decode kernel: X, W, W_scale and their row pitches must be 16-byte aligned");
  if (d.c_dtype != MX_F32 && d.c_dtype != MX_BF16) return set_error(MX_ERR_DTYPE, "decode kernel: bad output dtype");
  const int tiles = d.N / 16;
  int grid = tiles < 256 ? tiles : 256;
  if (grid == 0) return MX_OK;
  if (d.x_fmt == MX_E4M3) return launch_decode_x<MX_E4M3>(d, grid, stream);
  return launch_decode_x<MX_E5M2>(d, grid, stream);
}

}  // namespace mx
