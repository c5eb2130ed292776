// Tile-level building blocks shared by the scaled-MFMA GEMM kernels (gfx950): tile configuration,
// buffer descriptors, LDS swizzle, MFMA fragment loads and the output store.
#pragma once
#include "mx_common.h"

namespace mx {

typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(3))) const v4i lds_v4i;

constexpr uint32_t kOobOffset = 0x80000000u;  // beyond num_records of every descriptor we build

template <int AF_, int BF_, int BM_, int BN_, int WGM_, int WGN_>
struct Cfg {
  static constexpr int AF = AF_, BF = BF_, BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
  static constexpr int NW = WGM * WGN, NT = NW * 64;
  static constexpr int A_EB = (AF == MX_E2M1) ? 4 : 8, B_EB = (BF == MX_E2M1) ? 4 : 8;
  // MFMA K-steps (128 elements) per LDS stage: two when both operands are 4-bit so that a stage row
  // is still 128 bytes
  static constexpr int KSUB = (A_EB == 4 && B_EB == 4) ? 2 : 1;
  static constexpr int BKE = 128 * KSUB;
  static constexpr int A_RB = BKE * A_EB / 8, B_RB = BKE * B_EB / 8;   // bytes per stage row
  static constexpr int A_CPR = A_RB / 16, B_CPR = B_RB / 16;           // 16-byte chunks per row
  static constexpr int A_STAGE = BM * A_RB, B_STAGE = BN * B_RB, STAGE = A_STAGE + B_STAGE;
  static constexpr int LDS_BYTES = 2 * STAGE;
  static constexpr int A_LOADS = BM * A_CPR / NT, B_LOADS = BN * B_CPR / NT;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;   // wave tile
  static constexpr int MT = WTM / 16, NTL = WTN / 16;    // 16x16 MFMA tiles per wave
  static_assert(WTM % 64 == 0 && WTN % 64 == 0, "wave tile must cover whole 64-row scale groups");
  static_assert((BM * A_CPR) % NT == 0 && (BN * B_CPR) % NT == 0, "loads must divide evenly");
  static_assert(A_CPR == 8 || A_CPR == 4, "row is 64 or 128 bytes");
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// swizzle term of a tile row: chunk c of row R lives at chunk position c ^ swz<CPR>(R)
template <int CPR>
__device__ inline int swz(int row) {
  return (row / (16 / CPR)) % CPR;
}

// LDS swizzle of the B rows for that read pattern: built from the row bits that tell the 16 lanes of a read
// apart beyond the bank half (CPR = 8: bits 1, 3, 4; CPR = 4: bits 3, 4); for row bperm_row(j, c) it equals
// swz<CPR>(c), whatever j is.
template <int CPR>
__device__ inline int swz_bperm(int row) {
  if constexpr (CPR == 8) return ((row >> 1) & 1) | (((row >> 3) & 3) << 1);
  else return (row >> 3) & (CPR - 1);
}

// Fragment of one 16-row tile for MFMA K-step kk of the stage, lane group gq, in the operand layout
// described at the top of the file.  8-bit formats: two 16-byte chunks; 4-bit: one, in the low dwords.
template <int RB, int EB>
__device__ inline v8i load_frag(lds_u8* tile, int row, int kk, int gq, int sw) {
  if constexpr (EB == 8) {
    const int c = kk * 8 + gq;   // bytes 16 g .. 16 g + 15 and 64 + 16 g .. of the 128-byte K-step
    const v4i lo = *(lds_v4i*)(tile + row * RB + ((c ^ sw) << 4));
    const v4i hi = *(lds_v4i*)(tile + row * RB + (((c + 4) ^ sw) << 4));
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  } else {
    const int c = kk * 4 + gq;
    const v4i lo = *(lds_v4i*)(tile + row * RB + ((c ^ sw) << 4));
    return (v8i){lo.x, lo.y, lo.z, lo.w, 0, 0, 0, 0};
  }
}

// One scaled MFMA; the B fragment's scales are byte `bsel` of bscale, the A fragment's byte `asel` of ascale (in the
// native scale layout a register holds one K-step's scales of four 16-row tiles, so the byte is the tile's index in
// its group of four).  bsel and asel must fold to constants: the instruction encodes them.
template <int BFMT, int AFMT>
__device__ __forceinline__ v4f mfma_scaled(const v8i& bfrag, const v8i& afrag, const v4f& acc, int bsel, int bscale,
                                           int asel, int ascale) {
#define MX_MFMA_CASE(SB, SA)                                                                                   \
  case SB * 4 + SA:                                                                                            \
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bfrag, afrag, acc, BFMT, AFMT, SB, bscale, SA, ascale);
  switch (bsel * 4 + asel) {
    MX_MFMA_CASE(0, 0) MX_MFMA_CASE(0, 1) MX_MFMA_CASE(0, 2) MX_MFMA_CASE(0, 3)
    MX_MFMA_CASE(1, 0) MX_MFMA_CASE(1, 1) MX_MFMA_CASE(1, 2) MX_MFMA_CASE(1, 3)
    MX_MFMA_CASE(2, 0) MX_MFMA_CASE(2, 1) MX_MFMA_CASE(2, 2) MX_MFMA_CASE(2, 3)
    MX_MFMA_CASE(3, 0) MX_MFMA_CASE(3, 1) MX_MFMA_CASE(3, 2) MX_MFMA_CASE(3, 3)
  }
#undef MX_MFMA_CASE
  __builtin_unreachable();
}

template <typename OutT>
__device__ inline void store4(OutT* p, const v4f& v, bool accumulate, int nvalid, bool vec_ok);

template <>
__device__ inline void store4<float>(float* p, const v4f& v, bool accumulate, int nvalid,
                                     bool vec_ok) {
  if (nvalid >= 4 && vec_ok) {
    v4f o = v;
    if (accumulate) o += *(const v4f*)p;
    *(v4f*)p = o;
  } else {
    for (int e = 0; e < 4; ++e)
      if (e < nvalid) p[e] = accumulate ? p[e] + v[e] : v[e];
  }
}

template <>
__device__ inline void store4<uint16_t>(uint16_t* p, const v4f& v, bool accumulate, int nvalid,
                                        bool vec_ok) {
  if (nvalid >= 4 && vec_ok) {
    v4f o = v;
    if (accumulate) {
      const uint2 old = *(const uint2*)p;
      o.x += bf16_to_f32((uint16_t)old.x);
      o.y += bf16_to_f32((uint16_t)(old.x >> 16));
      o.z += bf16_to_f32((uint16_t)old.y);
      o.w += bf16_to_f32((uint16_t)(old.y >> 16));
    }
    uint2 w;
    w.x = (uint32_t)f32_to_bf16(o.x) | ((uint32_t)f32_to_bf16(o.y) << 16);
    w.y = (uint32_t)f32_to_bf16(o.z) | ((uint32_t)f32_to_bf16(o.w) << 16);
    *(uint2*)p = w;
  } else {
    for (int e = 0; e < 4; ++e)
      if (e < nvalid) p[e] = f32_to_bf16(accumulate ? bf16_to_f32(p[e]) + v[e] : v[e]);
  }
}

// four consecutive outputs, no bounds, alignment or accumulate handling (interior tiles)
template <typename OutT>
__device__ inline void store4_full(OutT* p, const v4f& v);

template <>
__device__ inline void store4_full<float>(float* p, const v4f& v) {
  *(v4f*)p = v;
}

template <>
__device__ inline void store4_full<uint16_t>(uint16_t* p, const v4f& v) {
  // v_cvt_pk_bf16_f32: round to nearest even, the same result as f32_to_bf16 for every non-NaN input
  typedef float f2 __attribute__((ext_vector_type(2)));
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  uint2 w;
  w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((f2){v.x, v.y}, b2));
  w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((f2){v.z, v.w}, b2));
  *(uint2*)p = w;
}

// eight consecutive outputs (two accumulator quads), no bounds, alignment or accumulate handling
template <typename OutT>
__device__ inline void store8_full(OutT* p, const v4f& v0, const v4f& v1);

template <>
__device__ inline void store8_full<float>(float* p, const v4f& v0, const v4f& v1) {
  *(v4f*)p = v0;
  *(v4f*)(p + 4) = v1;
}

template <>
__device__ inline void store8_full<uint16_t>(uint16_t* p, const v4f& v0, const v4f& v1) {
  typedef float f2 __attribute__((ext_vector_type(2)));
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  u4 w;
  w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((f2){v0.x, v0.y}, b2));
  w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((f2){v0.z, v0.w}, b2));
  w.z = __builtin_bit_cast(uint32_t, __builtin_convertvector((f2){v1.x, v1.y}, b2));
  w.w = __builtin_bit_cast(uint32_t, __builtin_convertvector((f2){v1.z, v1.w}, b2));
  *(u4*)p = w;
}

}  // namespace mx
