// Shared definitions for the libmxgemm kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxgemm.h"

namespace mx {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// ---- error reporting (host) ------------------------------------------------------------------
int set_error(int code, const char* fmt, ...);

// ---- native scale layouts ----------------------------------------------------------------------
// Both hold 16 bytes per (64-row group G, K-quad Q of four 128-element MFMA K-steps, lane), stored [G][Q][lane]:
// a 4 x 4 byte matrix of the scales of four rows for the four K-steps of the quad, for the 32-element K block
// (4 Q + t) * 4 + lane / 16 of K-step t.  One 16-byte load per lane (1 KiB contiguous per wave) brings a group's
// scales for a quad.  Rows are padded to a multiple of 64 and K-steps to a multiple of 4 with the byte 127 (1.0).
//   MX_SCALE_NATIVE (kernels on the 16x16x128 instruction): dword t = K-step, byte b = row, so that one register
//     feeds the four 16-row tiles of a group for one K-step (the tile is picked by the instruction's byte select).
//       A operand (kPackA): byte b = row 64 G + 16 b + lane % 16
//       B operand (kPackB): byte b = row 64 G + bperm_row(b, lane % 16), the row order in which the kernels feed
//                           B to the instruction
//   MX_SCALE_NATIVE32 (kernels on the 32x32x64 instruction, kPackTile32): dword b = row 64 G + 16 b + lane % 16,
//     byte t = K-step; both operands alike.
enum { kPackA = 0, kPackB = 1, kPackTile32 = 2 };
// ---- column order of the 16x16x128 kernels' B fragments ------------------------------------------------
// MFMA tile j (0..3) of a wave's 64 B rows takes, as its operand row c, B row
//     bperm_row(j, c) = 32 (j / 2) + 8 (c / 4) + 4 (j % 2) + c % 4
// instead of 16 j + c.  Lane (c, g) of the result then holds columns 32 (j / 2) + 8 g + 4 (j % 2) + e,
// e = 0..3: the tiles j = 2p and 2p + 1 give it 8 consecutive outputs, which leave as one 16-byte (bf16) or
// two adjacent 16-byte (fp32) stores -- half as many store instructions as with 4 consecutive outputs.
__host__ __device__ inline int bperm_tile_off(int j) { return 32 * (j >> 1) + 4 * (j & 1); }   // part of the row that depends on j
__host__ __device__ inline int bperm_lane_off(int c) { return 8 * (c >> 2) + (c & 3); }         // part that depends on the lane
__host__ __device__ inline int bperm_row(int j, int c) { return bperm_tile_off(j) + bperm_lane_off(c); }

__host__ __device__ inline int64_t packed_scale_quads(int64_t K) { return (K + 511) / 512; }
__host__ __device__ inline int64_t packed_scale_dwords(int64_t rows, int64_t K) {
  return ((rows + 63) / 64) * packed_scale_quads(K) * 256;
}

// ---- element decode (device) -------------------------------------------------------------------
__device__ inline float decode_e8m0(uint32_t b) {
  // 2^(b-127); 0xFF -> NaN; b == 0 -> 2^-127 (an fp32 subnormal, bit pattern 0x00400000)
  if (b == 0xFF) return __builtin_nanf("");
  uint32_t bits = b ? (b << 23) : 0x00400000u;
  return __builtin_bit_cast(float, bits);
}

__device__ inline float decode_e4m3(uint32_t c) {
  uint32_t e = (c >> 3) & 0xF, m = c & 7;
  float v;
  if ((c & 0x7F) == 0x7F) {
    v = __builtin_nanf("");
  } else if (e == 0) {
    v = (float)m * 0.001953125f;  // m * 2^-9
  } else {
    v = __builtin_bit_cast(float, ((e + 120u) << 23) | (m << 20));
  }
  return (c & 0x80) ? -v : v;
}

__device__ inline float decode_e5m2(uint32_t c) {
  // E5M2 is the upper byte of an IEEE half
  _Float16 h = __builtin_bit_cast(_Float16, (uint16_t)(c << 8));
  return (float)h;
}

__device__ inline float decode_e2m1(uint32_t c) {
  uint32_t e = (c >> 1) & 3, m = c & 1;
  float v = e == 0 ? 0.5f * (float)m : __builtin_bit_cast(float, ((e + 126u) << 23) | (m << 22));
  return (c & 8) ? -v : v;
}

__device__ inline float decode_elem(uint32_t c, int fmt) {
  return fmt == MX_E4M3 ? decode_e4m3(c) : fmt == MX_E5M2 ? decode_e5m2(c) : decode_e2m1(c);
}

// ---- fp32 -> bf16 bits, round to nearest even (torch's .to(bfloat16)) ---------------------------
__device__ inline uint16_t f32_to_bf16(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ inline float bf16_to_f32(uint16_t h) {
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}

// ---- launchers implemented in the kernel translation units ---------------------------------------
struct GemmArgs {
  const uint8_t* A;        // [M rows][lda bytes], K contiguous
  const uint8_t* B;        // [N rows][ldb bytes], K contiguous (i.e. the column-major K x N operand)
  const uint32_t* As;      // native packed scales of A rows
  const uint32_t* Bs;      // native packed scales of B rows (per expert when grouped)
  void* C;
  int64_t lda, ldb, ldc;   // lda/ldb in bytes, ldc in elements
  int32_t M, N, K;         // K in elements
  int32_t a_fmt, b_fmt, c_dtype, accumulate;
  // grouped (MoE) extension; sorted_token_ids == nullptr for the plain GEMM
  const int32_t* sorted_token_ids;
  const int32_t* sorted_expert_ids;
  const float* topk_weights;
  int32_t tile_m, replicas;
  int32_t num_experts;       // entries of sorted_expert_ids are clamped to [0, num_experts)
  int64_t num_valid_ids;
  int64_t b_expert_stride;   // bytes between experts in B
  int64_t bs_expert_stride;  // dwords between experts in Bs
  int64_t a_rows;            // rows of the A tensor (for the buffer descriptor)
  int32_t stagger;           // 1: workgroups start their K walk at different quads
  // split-K (one-tile kernels only): K is the slice length, slice i reads the scales / writes the partial
  // output i strides further on
  int32_t k_splits;
  int64_t as_split_stride, bs_split_stride;   // dwords
  int64_t c_split_stride;                     // elements of C
};

int launch_gemm_mfma(const GemmArgs& g, int kernel_id, hipStream_t stream);
// A list of independent plain products (no grouping, no split-K, one element format pair and output dtype for the
// whole list) on the 128 x 128 one-tile kernel body: one persistent launch per 32 problems walks the concatenated
// tile list (the scheme of grouped_matmul_kernel, test/kernels/group_gemm.py:10-38).
int launch_gemm_mfma_list(const GemmArgs* problems, int n, hipStream_t stream);
int launch_gemm_pingpong(const GemmArgs& g, hipStream_t stream);
// the 32x32x64-instruction variant: 8-bit element formats only
bool pingpong32_supports(int a_fmt, int b_fmt);
int launch_gemm_pingpong32(const GemmArgs& g, hipStream_t stream);
// persistent four-wave kernel (128 x 128 per wave): plain products of 8-bit operands, K >= 384
bool gemm_w4_supports(const GemmArgs& g);
int launch_gemm_w4(const GemmArgs& g, hipStream_t stream);
// C[m, n] (+)= sum over `splits` fp32 partials [splits][M][N]; C fp32 or bf16 with row pitch ldc
int launch_splitk_reduce(const float* partials, int splits, int64_t M, int64_t N, void* C, int64_t ldc,
                         int c_dtype, int accumulate, hipStream_t stream);

struct GenericArgs {
  const uint8_t* A; const uint8_t* As; const uint8_t* B; const uint8_t* Bs; void* C;
  int32_t batch, M, N, K, block;
  int32_t a_fmt, b_fmt, scale_fmt, c_dtype, accumulate;
  int32_t a_packed_k, b_packed_k;       // E2M1: 1 if packed along K, 0 if packed along M (A) / N (B)
  int64_t a_sb, a_sm, a_sk;             // strides (bytes) of A over batch, M, K (packed dim: per byte)
  int64_t as_sb, as_sm, as_sk;
  int64_t b_sb, b_sk, b_sn;
  int64_t bs_sb, bs_sk, bs_sn;
  int64_t c_sb, c_sm, c_sn;             // elements
  int32_t as_layout, bs_layout;         // MX_SCALE_2D or MX_SCALE_SWIZZLE_32_4_4
  // grouped extension
  const int32_t* sorted_token_ids; const int32_t* sorted_expert_ids; const float* topk_weights;
  int32_t tile_m, replicas, num_experts; int64_t num_valid_ids; int64_t num_slots;
  int64_t b_se, bs_se;                  // expert strides (bytes)
};
int launch_gemm_generic(const GenericArgs& g, hipStream_t stream);

struct PackArgs {
  const uint8_t* src; uint32_t* dst;
  int64_t rows, K;               // logical rows and K elements
  int64_t s_batch, s_row, s_kb;  // byte strides of the 2-D source
  int32_t layout;                // MX_SCALE_2D / MX_SCALE_SWIZZLE_32_4_4
  int32_t batch;
  int32_t target;                // kPackA / kPackB / kPackTile32
  // optional row gather (grouped GEMM): row p reads source row idx[p] / replicas if idx[p] < num_valid
  const int32_t* gather_ids; int32_t replicas; int64_t num_valid_ids;
};
int launch_pack_scales(const PackArgs& p, hipStream_t stream);
// both operands of one GEMM in a single launch; either pointer may be null
int launch_pack_scales_pair(const PackArgs* a, const PackArgs* b, hipStream_t stream);
// any number of plain 2-D scale tensors (64 per launch)
int launch_pack_scales_list(const PackArgs* list, int n, hipStream_t stream);

struct QuantArgs {
  const void* x; uint8_t* xq; uint8_t* scale;
  int64_t rows, K, Kpad;
  int64_t x_ld, xq_ld, sc_ld;    // elements / bytes / bytes
  int32_t x_dtype, fmt, scale_mode;
  // fused producer: the value quantised is silu(x[row, k]) * up[row, k] (up has the dtype and pitch of x)
  const void* up;
};
int launch_quantize(const QuantArgs& q, hipStream_t stream);

// `counts`: moe_align_workspace_bytes(num_ids, num_experts) bytes of scratch (per-chunk histograms)
int64_t moe_align_workspace_bytes(int64_t num_ids, int32_t num_experts);
int launch_moe_align(const int32_t* topk_ids, int64_t num_ids, int32_t num_experts, int32_t tile_m,
                     int32_t* sorted_token_ids, int32_t* sorted_expert_ids, int32_t* num_slots_out,
                     int64_t max_slots, int32_t* counts, hipStream_t stream);

struct DecodeArgs {
  const uint8_t* X; const uint8_t* Xs; const uint8_t* W; const uint8_t* Ws; void* C;
  int32_t M, N, K;                 // M <= 32
  int64_t ldx, ldxs, ldw, ldws, ldc;
  int32_t x_fmt, w_fmt, c_dtype, accumulate;
};
int launch_gemm_decode(const DecodeArgs& d, hipStream_t stream);

}  // namespace mx
