// Layout-agnostic block-scaled matmul: one thread per output element, fp32 arithmetic.
//
// Covers everything the MFMA kernels do not: arbitrary strides (row-major K x N operands as in
// test/test_mma_scaled.py:82-100), FP4 packed along the non-K axis (test_mma_scaled.py:163-183),
// scaling block 16, E4M3 scale bytes for FP4 (src/cuda/tile/_datatype.py:482-489), a broadcast
// batch dimension (test_mma_scaled.py:128-145), swizzle_32_4_4 scale tensors read in place, and
// the gather/scatter structure of fused_moe_kernel (test/kernels/fused_moe.py:14-82).
// It is a correctness path, not a fast one.
#include "mx_common.h"

namespace mx {
namespace {

__device__ inline uint32_t load_code(const uint8_t* base, int fmt, int64_t off_major, int64_t s_major,
                                     int64_t idx_k, int64_t s_k, int64_t idx_other, int packed_k) {
  // returns the element code at (other = idx_other, k = idx_k); `off_major` already points at the
  // batch.  For E2M1 the packed axis holds two logical elements per byte (low nibble first).
  if (fmt != MX_E2M1) return base[off_major + idx_other * s_major + idx_k * s_k];
  if (packed_k) {
    const uint8_t b = base[off_major + idx_other * s_major + (idx_k >> 1) * s_k];
    return (idx_k & 1) ? (b >> 4) : (b & 0xF);
  }
  const uint8_t b = base[off_major + (idx_other >> 1) * s_major + idx_k * s_k];
  return (idx_other & 1) ? (b >> 4) : (b & 0xF);
}

__device__ inline int64_t swizzled_offset(int64_t row, int64_t kb, int64_t KB) {
  // flat offset of logical scale (row, kb) inside a contiguous swizzle_32_4_4 tensor
  // (test/kernels/kernel_utils.py:83-98): [row/128][kb/4][row%32][(row%128)/32][kb%4]
  const int64_t m0 = row >> 7, m2 = (row & 127) >> 5, m1 = row & 31, k0 = kb >> 2, k1 = kb & 3;
  return ((m0 * (KB >> 2) + k0) * 32 + m1) * 16 + m2 * 4 + k1;
}

__device__ inline float decode_scale(uint32_t b, int scale_fmt) {
  return scale_fmt == MX_E8M0 ? decode_e8m0(b) : decode_e4m3(b);
}

__global__ __launch_bounds__(256) void generic_kernel(const GenericArgs g) {
  const int64_t n = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t mrow = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  const int64_t b = blockIdx.z;
  const bool grouped = g.sorted_token_ids != nullptr;
  const int64_t Mlimit = grouped ? g.num_slots : g.M;
  if (mrow >= Mlimit || n >= g.N) return;

  int64_t arow = mrow, crow = mrow;
  int64_t boff = b * g.b_sb, bsoff = b * g.bs_sb;
  float w = 1.f;
  if (grouped) {
    const int id = g.sorted_token_ids[mrow];
    if (id < 0 || id >= g.num_valid_ids) return;
    arow = id / g.replicas;
    crow = id;
    int e = g.sorted_expert_ids[mrow / g.tile_m];
    e = e < 0 ? 0 : (e >= g.num_experts ? g.num_experts - 1 : e);   // never outside W
    boff = (int64_t)e * g.b_se;
    bsoff = (int64_t)e * g.bs_se;
    if (g.topk_weights) w = g.topk_weights[id];
  }
  const int64_t aoff = b * g.a_sb, asoff = b * g.as_sb;
  const int64_t KB = g.K / g.block;

  float acc = 0.f;
  for (int64_t kb = 0; kb < KB; ++kb) {
    float part = 0.f;
    for (int kk = 0; kk < g.block; ++kk) {
      const int64_t k = kb * g.block + kk;
      const uint32_t ca = load_code(g.A, g.a_fmt, aoff, g.a_sm, k, g.a_sk, arow, g.a_packed_k);
      // B is addressed as (k, n): "major" stride is over n
      const uint32_t cb = load_code(g.B, g.b_fmt, boff, g.b_sn, k, g.b_sk, n, g.b_packed_k);
      part = fmaf(decode_elem(ca, g.a_fmt), decode_elem(cb, g.b_fmt), part);
    }
    const uint8_t sa = g.as_layout == MX_SCALE_SWIZZLE_32_4_4
                           ? g.As[asoff + swizzled_offset(arow, kb, KB)]
                           : g.As[asoff + arow * g.as_sm + kb * g.as_sk];
    const uint8_t sb = g.bs_layout == MX_SCALE_SWIZZLE_32_4_4
                           ? g.Bs[bsoff + swizzled_offset(n, kb, KB)]
                           : g.Bs[bsoff + kb * g.bs_sk + n * g.bs_sn];
    acc += (part * decode_scale(sa, g.scale_fmt)) * decode_scale(sb, g.scale_fmt);
  }
  acc *= w;

  const int64_t ci = b * g.c_sb + crow * g.c_sm + n * g.c_sn;
  if (g.c_dtype == MX_F32) {
    float* c = (float*)g.C;
    c[ci] = g.accumulate ? c[ci] + acc : acc;
  } else {
    uint16_t* c = (uint16_t*)g.C;
    c[ci] = f32_to_bf16(g.accumulate ? bf16_to_f32(c[ci]) + acc : acc);
  }
}

}  // namespace

int launch_gemm_generic(const GenericArgs& g, hipStream_t stream) {
  const int64_t rows = g.sorted_token_ids ? g.num_slots : g.M;
  if (rows <= 0 || g.N <= 0 || g.batch <= 0) return MX_OK;
  const int64_t gy = (rows + 15) / 16;
  if (gy > 65535) return set_error(MX_ERR_SHAPE, "generic kernel: too many rows (%lld)", (long long)rows);
  dim3 grid((unsigned)((g.N + 15) / 16), (unsigned)gy, (unsigned)g.batch);
  hipLaunchKernelGGL(generic_kernel, grid, dim3(256), 0, stream, g);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "generic_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

}  // namespace mx
