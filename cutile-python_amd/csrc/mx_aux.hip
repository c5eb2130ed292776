// Memory-bound helpers around the block-scaled GEMM: MX quantisation, native scale re-layout and the
// MoE slot alignment.  All integer / byte work; results must be bit-exact.
#include "mx_common.h"

namespace mx {
namespace {

// ================================================================================================
// MX quantiser (replaces the torch-op chain of block_quantize, test/kernels/kernel_utils.py:38-80)
// ================================================================================================
// The shared exponent is computed on bit patterns.  Element conversion has two routes with identical
// results: the gfx950 scaled-conversion instructions for ordinary blocks, and an integer route (value =
// sig * 2^(ex-150) divided by 2^se by subtracting exponents, then rounded to nearest even onto the target
// grid in one step) for blocks with a zero / subnormal amax, inf / NaN or an extreme scale, where denormal
// modes or the instruction's special cases could otherwise change a bit.

struct Unpacked {
  uint32_t sig;   // 24-bit significand with the leading one at bit 23 (0 for zero)
  int ex;         // biased exponent such that value = sig * 2^(ex - 150)
  uint32_t sign;  // 0 or 1
  int cls;        // 0 finite, 1 inf, 2 nan
};

__device__ inline Unpacked unpack_f32(uint32_t bits) {
  Unpacked u;
  u.sign = bits >> 31;
  const uint32_t a = bits & 0x7FFFFFFFu;
  u.cls = a > 0x7F800000u ? 2 : (a == 0x7F800000u ? 1 : 0);
  int ex = (int)(a >> 23);
  uint32_t sig = a & 0x7FFFFFu;
  if (ex == 0) {
    if (sig != 0) {  // subnormal: normalise
      const int lz = __builtin_clz(sig) - 8;
      sig <<= lz;
      ex = 1 - lz;
    }
  } else {
    sig |= 0x800000u;
  }
  u.sig = sig;
  u.ex = ex;
  return u;
}

// round-to-nearest-even of sig / 2^sh, sh in [1, 31]
__device__ inline uint32_t rne_shift(uint32_t sig, int sh) {
  return (sig + ((1u << (sh - 1)) - 1u) + ((sig >> sh) & 1u)) >> sh;
}

// Generic minifloat encoder: MBITS mantissa bits, minimum normal exponent EMIN, exponent bias BIAS.
// Returns the magnitude code without clamping (may exceed the format's largest finite code).
template <int MBITS, int EMIN, int BIAS>
__device__ inline uint32_t encode_mag(const Unpacked& u, int se) {
  if (u.sig == 0) return 0;
  const int E = u.ex - 127 - se;            // exponent of x / 2^se
  const int Eq = E > EMIN ? E : EMIN;
  int sh = (23 - MBITS) + (Eq - E);
  if (sh > 31) sh = 31;                     // anything this small rounds to zero
  const uint32_t n = rne_shift(u.sig, sh);  // in units of 2^(Eq - MBITS); normal range: [2^MBITS, 2^(MBITS+1)]
  if (E > 300) return 0xFFFFu;              // cannot happen for finite fp32 / E8M0 scales; keeps shifts sane
  return (uint32_t)((Eq + BIAS - 1) << MBITS) + n;
}

__device__ inline uint32_t encode_e4m3(const Unpacked& u, int se, bool saturate) {
  const uint32_t s = u.sign << 7;
  if (u.cls == 2) return s | 0x7F;
  if (u.cls == 1) return s | (saturate ? 0x7Eu : 0x7Fu);
  uint32_t c = encode_mag<3, -6, 7>(u, se);
  if (c > 0x7E) c = saturate ? 0x7E : 0x7F;   // torch's cast: above 448 after rounding -> NaN
  return s | c;
}

__device__ inline uint32_t encode_e5m2(const Unpacked& u, int se, bool saturate) {
  const uint32_t s = u.sign << 7;
  if (u.cls == 2) return s | 0x7F;
  if (u.cls == 1) return s | (saturate ? 0x7Bu : 0x7Cu);
  uint32_t c = encode_mag<2, -14, 15>(u, se);
  if (c > 0x7B) c = saturate ? 0x7B : 0x7C;   // IEEE-like: overflow -> inf
  return s | c;
}

__device__ inline uint32_t encode_e2m1(const Unpacked& u, int se) {
  const uint32_t s = u.sign << 3;
  if (u.cls != 0) return s | 7;
  uint32_t c = encode_mag<1, 0, 1>(u, se);
  if (c > 7) c = 7;                           // finite-only format: clamp to +-6
  return s | c;
}

__device__ inline float load_as_f32(const void* p, int64_t i, int dtype) {
  if (dtype == MX_F32) return ((const float*)p)[i];
  if (dtype == MX_BF16) return bf16_to_f32(((const uint16_t*)p)[i]);
  return (float)((const _Float16*)p)[i];
}

// silu(a) * b = a / (1 + exp(-a)) * b as a fixed sequence of correctly rounded fp32 operations (no fused
// multiply-add, no approximate instruction), so that a host restatement with the same sequence gets the
// same bits: exp(-a) = 2^z, z = -a * log2(e) clamped to +-125, z = n + f with n = rint(z), 2^f by the
// degree-7 Taylor polynomial in f * ln 2 (|f| <= 0.5: truncation error below 1e-8), scaled by 2^n exactly.
__device__ inline float silu_mul_f32(float a, float b) {
  float z = __fmul_rn(-a, 1.44269504f);
  z = fminf(fmaxf(z, -125.0f), 125.0f);
  const float n = __builtin_rintf(z);
  const float f = __fsub_rn(z, n);
  float p = 1.52527338e-5f;
  p = __fadd_rn(__fmul_rn(p, f), 1.54035304e-4f);
  p = __fadd_rn(__fmul_rn(p, f), 1.33335581e-3f);
  p = __fadd_rn(__fmul_rn(p, f), 9.61812911e-3f);
  p = __fadd_rn(__fmul_rn(p, f), 5.55041087e-2f);
  p = __fadd_rn(__fmul_rn(p, f), 2.40226507e-1f);
  p = __fadd_rn(__fmul_rn(p, f), 6.93147181e-1f);
  p = __fadd_rn(__fmul_rn(p, f), 1.0f);
  const float e = __fmul_rn(p, __builtin_bit_cast(float, (uint32_t)((int)n + 127) << 23));
  const float s = __fdiv_rn(1.0f, __fadd_rn(1.0f, e));
  const float t = a < -87.5f ? 0.0f : __fmul_rn(a, s);   // exp(-a) is past the clamp: the true value is below 2^-120
  return __fmul_rn(t, b);
}

// EPL consecutive elements starting at element index i (all of them inside K checked by the caller for `vec`)
template <int EPL>
__device__ inline void load_as_f32_vec(const void* p, int64_t i, int dtype, bool vec, int nvalid, float* v) {
  if (vec && dtype == MX_F32) {
#pragma unroll
    for (int h = 0; h < EPL / 4; ++h) {
      const v4f t = *(const v4f*)((const float*)p + i + 4 * h);
      v[4 * h + 0] = t.x; v[4 * h + 1] = t.y; v[4 * h + 2] = t.z; v[4 * h + 3] = t.w;
    }
  } else if (vec && dtype == MX_BF16) {
    uint32_t t[EPL / 2];
    if constexpr (EPL >= 8) {
#pragma unroll
      for (int h = 0; h < EPL / 8; ++h) {
        const v4i r = *(const v4i*)((const uint16_t*)p + i + 8 * h);
        t[4 * h + 0] = (uint32_t)r.x; t[4 * h + 1] = (uint32_t)r.y; t[4 * h + 2] = (uint32_t)r.z; t[4 * h + 3] = (uint32_t)r.w;
      }
    } else {
      const uint2 r = *(const uint2*)((const uint16_t*)p + i);
      t[0] = r.x; t[1] = r.y;
    }
#pragma unroll
    for (int h = 0; h < EPL / 2; ++h) {
      v[2 * h] = bf16_to_f32((uint16_t)t[h]);
      v[2 * h + 1] = bf16_to_f32((uint16_t)(t[h] >> 16));
    }
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) v[e] = e < nvalid ? load_as_f32(p, i + e, dtype) : 0.f;
  }
}

// Where unit `gid` lives: 32 / EPL consecutive units are one 32-element block, EPL consecutive elements per unit.
struct QuantUnit {
  int64_t row, kb, k0;
  int sub;
  bool live;
};

template <int EPL>
__device__ inline QuantUnit quant_unit(const QuantArgs& q, int64_t gid) {
  constexpr int UPB = 32 / EPL;   // units (lanes) per block
  const int64_t KB = q.Kpad / 32;
  QuantUnit u;
  const int64_t blk = gid / UPB;
  u.sub = (int)(gid % UPB);
  u.live = blk < q.rows * KB;
  if (q.rows * KB < ((int64_t)1 << 31)) {   // uniform: 32-bit division is several times cheaper
    const uint32_t b32 = u.live ? (uint32_t)blk : 0u, kb32 = (uint32_t)KB;
    u.row = b32 / kb32;
    u.kb = b32 - (uint32_t)u.row * kb32;
  } else {
    u.row = u.live ? blk / KB : 0;
    u.kb = u.live ? blk % KB : 0;
  }
  u.k0 = u.kb * 32 + u.sub * EPL;
  return u;
}

// the (at most) EPL input values of a unit; the fused producer applies silu(x) * up
template <int EPL>
__device__ inline void quant_load(const QuantArgs& q, const QuantUnit& u, float* v, float* w) {
#pragma unroll
  for (int e = 0; e < EPL; ++e) v[e] = w[e] = 0.f;
  if (!u.live) return;
  const int64_t base = u.row * q.x_ld + u.k0;
  const int esz = q.x_dtype == MX_F32 ? 4 : 2;
  const int nvalid = q.K - u.k0 >= EPL ? EPL : (q.K > u.k0 ? (int)(q.K - u.k0) : 0);
  // 16-byte loads: fp32 in EPL / 4 pieces, bf16 as one (EPL = 8) or an 8-byte one (EPL = 4)
  const int align = (q.x_dtype == MX_F32 || EPL >= 8) ? 16 : 8;
  const bool vec = nvalid == EPL && q.x_dtype != MX_F16 &&
                   ((((uintptr_t)q.x) | ((uintptr_t)q.up) | (uintptr_t)(q.x_ld * esz)) & (align - 1)) == 0;
  load_as_f32_vec<EPL>(q.x, base, q.x_dtype, vec, nvalid, v);
  if (q.up) load_as_f32_vec<EPL>(q.up, base, q.x_dtype, vec, nvalid, w);
}

template <int EPL>
__device__ inline void quant_store(const QuantArgs& q, const QuantUnit& u, float* v, const float* w) {
  constexpr int UPB = 32 / EPL;
  const bool live = u.live;
  const int64_t row = u.row, kb = u.kb, k0 = u.k0;
  const int sub = u.sub;
  if (q.up) {
    const int nvalid = q.K - k0 >= EPL ? EPL : (q.K > k0 ? (int)(q.K - k0) : 0);
#pragma unroll
    for (int e = 0; e < EPL; ++e) v[e] = (live && e < nvalid) ? silu_mul_f32(v[e], w[e]) : 0.f;
  }
  // amax over the block on |bits| (monotone in |x| for finite values; NaN patterns compare largest)
  uint32_t bits[EPL], am = 0;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    bits[e] = __builtin_bit_cast(uint32_t, v[e]);
    const uint32_t a = bits[e] & 0x7FFFFFFFu;
    am = a > am ? a : am;
  }
#pragma unroll
  for (int d = 1; d < UPB; d <<= 1) {
    const uint32_t o = (uint32_t)__shfl_xor((int)am, d);
    am = o > am ? o : am;
  }

  // shared exponent
  int se;
  if (q.scale_mode == 0) {
    // reference rule: 2^ceil(log2(max(amax/448, 1e-12))), ceiling taken exactly on the fp32 quotient
    // (a block with an inf or NaN amax never uses this exponent: see nonfinite_ceil below)
    float t = __fdiv_rn(__builtin_bit_cast(float, am), 448.0f);
    t = t > 1e-12f ? t : 1e-12f;
    const uint32_t tb = __builtin_bit_cast(uint32_t, t);
    se = (int)(tb >> 23) - 127 + ((tb & 0x7FFFFFu) ? 1 : 0);
  } else {
    // OCP MX v1.0: floor(log2 amax) - emax_elem; all-zero block -> smallest scale
    const int emax = q.fmt == MX_E4M3 ? 8 : (q.fmt == MX_E5M2 ? 15 : 2);
    if (am == 0) {
      se = -127;
    } else {
      const int ex = (int)(am >> 23);
      const int fl = ex ? ex - 127 : (31 - __builtin_clz(am)) - 149;
      se = fl - emax;
    }
  }
  se = se < -127 ? -127 : (se > 127 ? 127 : se);
  const bool saturate = q.scale_mode != 0;

  // Reference rule with a non-finite amax: torch.clamp(min=) keeps NaN and inf / 448 stays inf, so the scale is
  // NaN or inf, both of which the cast to float8_e8m0fnu writes as 0xFF; x / scale is then NaN for every
  // element of a NaN block (the element's own sign if it is a NaN itself), and for an inf block NaN where
  // |x| is inf (inf / inf is the default NaN, whose sign bit is set on the hosts the reference runs on) and a
  // signed zero elsewhere.  E2M1 has no NaN: non-finite elements saturate to +-6 as in the finite case.
  const bool nonfinite_ceil = q.scale_mode == 0 && am >= 0x7F800000u;
  uint32_t code[EPL];
  if (nonfinite_ceil) {
    const bool blk_nan = am > 0x7F800000u;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const uint32_t a = bits[e] & 0x7FFFFFFFu, sgn = bits[e] >> 31;
      if (q.fmt == MX_E2M1) code[e] = (sgn << 3) | ((blk_nan || a == 0x7F800000u) ? 7u : 0u);
      else if (a > 0x7F800000u) code[e] = (sgn << 7) | 0x7Fu;
      else if (blk_nan) code[e] = 0x7Fu;
      else if (a == 0x7F800000u) code[e] = 0xFFu;
      else code[e] = sgn << 7;
    }
  } else
  // Blocks whose amax is a normal finite number and whose scale 2^se is a normal float take the hardware
  // scaled conversions (v_cvt_scalef32_pk_*: x / 2^se rounded to nearest even; FP8 overflows to NaN / inf,
  // FP4 saturates -- measured on MI355X against the integer encoders below for 270 k inputs per format).
  // The saturating FP8 rule clamps the magnitude to max_normal * 2^se first, which is exact.  Everything
  // else (zero or subnormal amax, inf / NaN, extreme scales) goes through the integer encoders.
  if (am >= 0x00800000u && am < 0x7F800000u && se > -127 && se < 120) {
    typedef short s2 __attribute__((ext_vector_type(2)));
    const float sc = __builtin_bit_cast(float, (uint32_t)(se + 127) << 23);
    float x[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) x[e] = v[e];
    if (saturate && q.fmt != MX_E2M1) {
      const float lim = __fmul_rn(q.fmt == MX_E4M3 ? 448.0f : 57344.0f, sc);
#pragma unroll
      for (int e = 0; e < EPL; ++e) x[e] = __builtin_copysignf(fminf(__builtin_fabsf(x[e]), lim), x[e]);
    }
#pragma unroll
    for (int h = 0; h < EPL / 4; ++h) {   // four elements at a time
      uint32_t packed;
      if (q.fmt == MX_E4M3) {
        s2 r = {0, 0};
        r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(r, x[4 * h + 0], x[4 * h + 1], sc, false);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(r, x[4 * h + 2], x[4 * h + 3], sc, true);
        packed = __builtin_bit_cast(uint32_t, r);
      } else if (q.fmt == MX_E5M2) {
        s2 r = {0, 0};
        r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(r, x[4 * h + 0], x[4 * h + 1], sc, false);
        r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(r, x[4 * h + 2], x[4 * h + 3], sc, true);
        packed = __builtin_bit_cast(uint32_t, r);
      } else {
        uint32_t r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, x[4 * h + 0], x[4 * h + 1], sc, 0);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, x[4 * h + 2], x[4 * h + 3], sc, 1);
        packed = (r & 0xFu) | ((r & 0xF0u) << 4) | ((r & 0xF00u) << 8) | ((r & 0xF000u) << 12);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) code[4 * h + e] = (packed >> (8 * e)) & 0xFFu;
    }
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const Unpacked un = unpack_f32(bits[e]);
      code[e] = q.fmt == MX_E4M3 ? encode_e4m3(un, se, saturate)
                : q.fmt == MX_E5M2 ? encode_e5m2(un, se, saturate)
                                   : encode_e2m1(un, se);
    }
  }
  if (!live) return;
  if (q.fmt == MX_E2M1) {
    // low nibble = even element (test/test_mma_scaled.py:155-160)
    uint8_t* out = q.xq + row * q.xq_ld + (k0 >> 1);
    constexpr int NB = EPL / 2;   // output bytes
    uint32_t word[(NB + 3) / 4] = {};
#pragma unroll
    for (int e = 0; e < NB; ++e) word[e / 4] |= (code[2 * e] | (code[2 * e + 1] << 4)) << (8 * (e % 4));
    if (NB >= 4 && ((((uintptr_t)q.xq) | (uintptr_t)q.xq_ld) & (NB - 1)) == 0) {
      if constexpr (NB == 8) *(uint2*)out = make_uint2(word[0], word[1]);
      else *(uint32_t*)out = word[0];
    } else {
#pragma unroll
      for (int e = 0; e < NB; ++e) out[e] = (uint8_t)(word[e / 4] >> (8 * (e % 4)));
    }
  } else {
    uint8_t* out = q.xq + row * q.xq_ld + k0;
    uint32_t word[EPL / 4];
#pragma unroll
    for (int h = 0; h < EPL / 4; ++h)
      word[h] = code[4 * h] | (code[4 * h + 1] << 8) | (code[4 * h + 2] << 16) | (code[4 * h + 3] << 24);
    if ((((((uintptr_t)q.xq) | (uintptr_t)q.xq_ld) & (EPL - 1))) == 0) {
      if constexpr (EPL == 16) *(uint4*)out = make_uint4(word[0], word[1], word[2], word[3]);
      else if constexpr (EPL == 8) *(uint2*)out = make_uint2(word[0], word[1]);
      else *(uint32_t*)out = word[0];
    } else {
#pragma unroll
      for (int e = 0; e < EPL; ++e) out[e] = (uint8_t)code[e];
    }
  }
  if (sub == 0) q.scale[row * q.sc_ld + kb] = nonfinite_ceil ? (uint8_t)0xFF : (uint8_t)(se + 127);
}

// 32 / EPL lanes per 32-element block, EPL consecutive elements per lane (8: half as many threads, and the
// per-block work -- the amax exchange, the shared exponent, the scale byte -- is spread over twice as many
// elements; 16-byte loads also from bf16 input); every thread handles kQuantUnroll units a grid apart and
// requests all their inputs before it processes the first (memory-level parallelism).
constexpr int kQuantUnroll = 2;
constexpr int kQuantEpl = 8;    // 16 measured no faster (58 -> 60 us on 8192^2 fp32)
template <int EPL>
__global__ __launch_bounds__(256) void quantize_kernel(const QuantArgs q) {
  const int64_t nthreads = (int64_t)gridDim.x * 256;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  QuantUnit u[kQuantUnroll];
  float v[kQuantUnroll][EPL], w[kQuantUnroll][EPL];
#pragma unroll
  for (int i = 0; i < kQuantUnroll; ++i) {
    u[i] = quant_unit<EPL>(q, gid + i * nthreads);
    quant_load<EPL>(q, u[i], v[i], w[i]);
  }
#pragma unroll
  for (int i = 0; i < kQuantUnroll; ++i) quant_store<EPL>(q, u[i], v[i], w[i]);
}

// ================================================================================================
// Native scale re-layout (see mx_common.h for the layout)
// ================================================================================================
// One workgroup re-lays out 64 rows x 4 K-quads (64 scale bytes per row) of one operand: the bytes are
// staged in LDS with whichever axis is contiguous in the source mapped to consecutive lanes (16-byte
// loads when alignment allows), then every thread assembles the four dwords of one (quad, lane) and
// writes them with one 16-byte store.  Up to two operands (A and B scales of one GEMM) share a launch.
struct PackPair {
  PackArgs p[2];
  int32_t blocks0;   // workgroups that belong to p[0]
};

__device__ inline int64_t scale_src_offset(const PackArgs& p, int64_t srow, int64_t kb, int64_t KB) {
  if (p.layout == MX_SCALE_SWIZZLE_32_4_4) {
    const int64_t m0 = srow >> 7, m2 = (srow & 127) >> 5, m1 = srow & 31, k0 = kb >> 2, k1 = kb & 3;
    return ((m0 * (KB >> 2) + k0) * 32 + m1) * 16 + m2 * 4 + k1;
  }
  return srow * p.s_row + kb * p.s_kb;
}

// up to kPackListMax plain 2-D scale tensors (the operands of a list of problems) in one launch; the entries are
// kept small so that the table travels as a kernel argument
constexpr int kPackListMax = 64;
struct PackEntry {
  const uint8_t* src; uint32_t* dst;
  int64_t rows, K, s_row, s_kb;
  int32_t target;
};
struct PackList {
  PackEntry p[kPackListMax];
  int32_t first_block[kPackListMax + 1];   // workgroups [first_block[i], first_block[i + 1]) belong to p[i]
  int32_t n;
};

__device__ inline void pack_scales_block(const PackArgs& p, const int64_t blk) {
  constexpr int LD = 68;   // LDS row pitch (bytes): 64 scale bytes + 4 so that rows start on distinct banks
  __shared__ __attribute__((aligned(16))) uint8_t tile[64 * LD];
  const int64_t KB = p.K / 32;
  const int64_t KQ = packed_scale_quads(p.K);
  const int64_t qgroups = (KQ + 3) / 4, rgroups = (p.rows + 63) / 64;
  const int64_t b = blk / (qgroups * rgroups);
  const int64_t t64 = (blk / qgroups) % rgroups;
  const int64_t Q0 = (blk % qgroups) * 4;
  const int tid = threadIdx.x;
  const uint8_t* src = p.src + b * p.s_batch;
  const int64_t row0 = t64 * 64, kb0 = Q0 * 16;

  // ---- stage 64 rows x 64 scale bytes; 127 (1.0) wherever the source has nothing -------------------------
  const bool plain = p.layout == MX_SCALE_2D && !p.gather_ids;
  if (plain && p.s_row == 1 && p.s_kb != 1) {
    // rows contiguous in the source: thread = (kb, 16 consecutive rows)
    const int kbi = tid >> 2, c = tid & 3;
    const int64_t kb = kb0 + kbi, r0 = row0 + c * 16;
    alignas(16) uint8_t v[16];
    const uint8_t* s = src + kb * p.s_kb + r0;
    if (kb < KB && r0 + 16 <= p.rows && (((uintptr_t)s) & 15) == 0) {
      *(uint4*)v = *(const uint4*)s;
    } else {
      for (int e = 0; e < 16; ++e) v[e] = (kb < KB && r0 + e < p.rows) ? s[e] : 127;
    }
    for (int e = 0; e < 16; ++e) tile[(c * 16 + e) * LD + kbi] = v[e];
  } else {
    // thread = (row, 16 consecutive K blocks)
    const int rowi = tid >> 2, c = tid & 3;
    const int64_t row = row0 + rowi, kb = kb0 + c * 16;
    int64_t srow = row;
    bool ok = row < p.rows;
    if (p.gather_ids) {
      const int id = ok ? p.gather_ids[row] : -1;
      ok = ok && id >= 0 && id < p.num_valid_ids;
      srow = id / p.replicas;
    }
    alignas(16) uint8_t v[16];
    const uint8_t* s = src + srow * p.s_row + kb;
    if (ok && p.layout == MX_SCALE_2D && p.s_kb == 1 && kb + 16 <= KB && (((uintptr_t)s) & 15) == 0) {
      *(uint4*)v = *(const uint4*)s;
    } else {
      for (int e = 0; e < 16; ++e) v[e] = (ok && kb + e < KB) ? src[scale_src_offset(p, srow, kb + e, KB)] : 127;
    }
    *(uint4*)(tile + rowi * LD + c * 16) = *(const uint4*)v;
  }
  __syncthreads();

  // ---- assemble: thread = (quad q of the group, lane): the 4 x 4 bytes (row, K-step) of the lane, K block
  // (4 (Q0 + q) + t) * 4 + lane / 16 for K-step t; which rows and which index is the dword depend on the target ---
  const int q = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
  if (Q0 + q >= KQ) return;
  uint32_t out[4];
  if (p.target == kPackTile32) {
    for (int i4 = 0; i4 < 4; ++i4) {
      const uint8_t* t = tile + (i4 * 16 + r) * LD + q * 16 + g;
      out[i4] = (uint32_t)t[0] | ((uint32_t)t[4] << 8) | ((uint32_t)t[8] << 16) | ((uint32_t)t[12] << 24);
    }
  } else {
    int row[4];
    for (int b = 0; b < 4; ++b) row[b] = p.target == kPackB ? bperm_row(b, r) : 16 * b + r;
    for (int t = 0; t < 4; ++t) {
      const uint8_t* c = tile + q * 16 + 4 * t + g;
      out[t] = (uint32_t)c[row[0] * LD] | ((uint32_t)c[row[1] * LD] << 8) | ((uint32_t)c[row[2] * LD] << 16) |
               ((uint32_t)c[row[3] * LD] << 24);
    }
  }
  uint32_t* dst = p.dst + b * packed_scale_dwords(p.rows, p.K) + ((t64 * KQ + Q0 + q) * 64 + lane) * 4;
  *(uint4*)dst = make_uint4(out[0], out[1], out[2], out[3]);
}

__global__ __launch_bounds__(256) void pack_scales_kernel(const PackPair pp) {
  const bool second = (int)blockIdx.x >= pp.blocks0;
  pack_scales_block(second ? pp.p[1] : pp.p[0], second ? blockIdx.x - pp.blocks0 : blockIdx.x);
}

__global__ __launch_bounds__(256) void pack_scales_list_kernel(const PackList pl) {
  int i = 0;
  while (i + 1 < pl.n && (int)blockIdx.x >= pl.first_block[i + 1]) ++i;   // uniform per workgroup
  const PackEntry& e = pl.p[i];
  PackArgs p = {};
  p.src = e.src; p.dst = e.dst; p.rows = e.rows; p.K = e.K; p.s_row = e.s_row; p.s_kb = e.s_kb;
  p.target = e.target;
  p.layout = MX_SCALE_2D; p.batch = 1; p.replicas = 1;
  pack_scales_block(p, (int)blockIdx.x - pl.first_block[i]);
}

// ================================================================================================
// MoE slot alignment (replaces moe_align_tile_size_torch, test/kernels/fused_moe.py:113-173)
// ================================================================================================
// A stable counting sort of the flattened expert ids over several workgroups, without atomics on global
// memory and without any slot written twice.  The ids are cut into B contiguous chunks, one per workgroup.
//   moe_hist_kernel (only when B > 1): workgroup b counts the ids of every expert in chunk b -> counts[b][e].
//   moe_place_kernel: workgroup b
//     1. sums column e of `counts` (thread e): ids of expert e in all chunks (total) and in the chunks before
//        its own (base); with B == 1 the totals come from its own counting pass instead;
//     2. exclusive scan of the tile-padded totals over the experts -> first slot of every expert (start);
//     3. places the ids of its chunk in order at start[e] + base[e] + (rank inside the chunk).  Up to 256
//        experts: every thread owns a contiguous segment of the chunk, per-thread per-expert counts live in
//        LDS as u16 (a chunk holds at most 65535 ids, so neither a count nor a prefix inside the chunk can
//        wrap) and become exclusive prefixes over the threads, which is what makes the order stable; more
//        experts: wave 0 walks the chunk 64 ids at a time and ranks equal experts with ballots;
//     4. experts b, b + B, ... : sentinel into the padding behind the expert's ids, expert id into its blocks;
//        all workgroups together: sentinel / expert 0 into the unused tail of the worst-case-sized outputs.
constexpr int kAlignThreads = 256;
constexpr int kAlignSegExperts = 256;      // up to this many experts the segment placement is used
constexpr int64_t kAlignMaxChunk = 65535;  // ids per workgroup (u16 prefixes inside a chunk)

__global__ __launch_bounds__(kAlignThreads) void moe_hist_kernel(const int32_t* __restrict__ topk_ids, int64_t n,
                                                                 int32_t E, int64_t chunk,
                                                                 int32_t* __restrict__ counts) {
  extern __shared__ int32_t sh[];   // [E]
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += kAlignThreads) sh[e] = 0;
  __syncthreads();
  const int64_t lo = (int64_t)blockIdx.x * chunk, hi = lo + chunk < n ? lo + chunk : n;
  for (int64_t i = lo + tid; i < hi; i += kAlignThreads) {
    const int e = topk_ids[i];
    if (e >= 0 && e < E) atomicAdd(&sh[e], 1);
  }
  __syncthreads();
  for (int e = tid; e < E; e += kAlignThreads) counts[(int64_t)blockIdx.x * E + e] = sh[e];
}

__global__ __launch_bounds__(kAlignThreads) void moe_place_kernel(const int32_t* __restrict__ topk_ids, int64_t n,
                                                                  int32_t E, int32_t tile_m, int64_t chunk,
                                                                  const int32_t* __restrict__ counts,
                                                                  int32_t* __restrict__ sorted_ids,
                                                                  int32_t* __restrict__ expert_ids,
                                                                  int32_t* __restrict__ num_slots_out,
                                                                  int64_t max_slots) {
  constexpr int T = kAlignThreads, LD = T + 2;   // row pitch 129 dwords: rows start on consecutive LDS banks
  extern __shared__ int32_t sh[];
  int32_t* total = sh;                  // [E] ids per expert
  int32_t* base = sh + E;               // [E] ids of the expert in earlier chunks; later the write cursor
  int32_t* start = sh + 2 * E;          // [E + 1] first slot of each expert
  int32_t* part = sh + 3 * E + 1;       // [T] partial sums of the scan
  uint16_t* cnt = (uint16_t*)(sh + 3 * E + 1 + T);   // [E][LD], segment placement only
  const int tid = threadIdx.x, B = gridDim.x, b = blockIdx.x;
  const bool seg_mode = E <= kAlignSegExperts;
  const int64_t lo = (int64_t)b * chunk, hi = lo + chunk < n ? lo + chunk : n;
  const int64_t seg = (hi - lo + T - 1) / T;
  const int64_t slo = lo + tid * seg < hi ? lo + tid * seg : hi, shi = slo + seg < hi ? slo + seg : hi;

  // ---- 1. totals and bases ------------------------------------------------------------------------------
  if (seg_mode) {
    for (int i = tid; i < E * LD / 2; i += T) ((uint32_t*)cnt)[i] = 0;
    __syncthreads();
    for (int64_t i = slo; i < shi; ++i) {
      const int e = topk_ids[i];
      if (e >= 0 && e < E) cnt[e * LD + tid] += 1;
    }
    __syncthreads();
    if (tid < E) {   // row e -> exclusive prefixes over the threads; the row sum is the chunk's count
      uint16_t* row = cnt + tid * LD;
      int32_t run = 0;
      for (int t = 0; t < T; ++t) {
        const int32_t c = row[t];
        row[t] = (uint16_t)run;
        run += c;
      }
      total[tid] = run;
    }
  } else if (B == 1) {
    for (int e = tid; e < E; e += T) total[e] = 0;
    __syncthreads();
    for (int64_t i = lo + tid; i < hi; i += T) {
      const int e = topk_ids[i];
      if (e >= 0 && e < E) atomicAdd(&total[e], 1);
    }
  }
  __syncthreads();
  for (int e = tid; e < E; e += T) {
    int32_t pre = 0;
    if (B > 1) {
      int32_t tot = 0;
      for (int bb = 0; bb < B; ++bb) {
        const int32_t c = counts[(int64_t)bb * E + e];
        if (bb < b) pre += c;
        tot += c;
      }
      total[e] = tot;
    }
    base[e] = pre;
  }
  __syncthreads();
  // ---- 2. first slot of every expert: thread t scans experts [t * per, (t + 1) * per) -------------------
  const int per = (E + T - 1) / T;
  {
    int32_t s2 = 0;
    for (int e = tid * per; e < (tid + 1) * per && e < E; ++e) s2 += (total[e] + tile_m - 1) / tile_m * tile_m;
    part[tid] = s2;
  }
  __syncthreads();
  if (tid == 0) {
    int32_t run = 0;
    for (int t = 0; t < T; ++t) {
      const int32_t c = part[t];
      part[t] = run;
      run += c;
    }
    start[E] = run;
    if (b == 0 && num_slots_out) *num_slots_out = run;
  }
  __syncthreads();
  {
    int32_t run = part[tid];
    for (int e = tid * per; e < (tid + 1) * per && e < E; ++e) {
      start[e] = run;
      run += (total[e] + tile_m - 1) / tile_m * tile_m;
    }
  }
  __syncthreads();
  // ---- 3. placement -------------------------------------------------------------------------------------
  if (seg_mode) {
    for (int64_t i = slo; i < shi; ++i) {
      const int e = topk_ids[i];
      if (e >= 0 && e < E) {
        const int32_t pos = start[e] + base[e] + cnt[e * LD + tid];
        cnt[e * LD + tid] += 1;
        sorted_ids[pos] = (int32_t)i;
      }
    }
  } else {
    for (int e = tid; e < E; e += T) base[e] += start[e];   // write cursor of this chunk
    __syncthreads();
    if (tid < 64) {
      for (int64_t i0 = lo; i0 < hi; i0 += 64) {
        const int64_t i = i0 + tid;
        int e = i < hi ? topk_ids[i] : -1;
        if (e >= E) e = -1;
        bool todo = e >= 0;
        while (__any(todo)) {
          const uint64_t pending = __ballot(todo);
          const int leader = __builtin_ctzll(pending);
          const int e0 = __shfl(e, leader);
          const bool mine = todo && e == e0;
          const uint64_t same = __ballot(mine);
          if (mine) {
            const int rank = __builtin_popcountll(same & ((1ull << tid) - 1ull));
            sorted_ids[base[e0] + rank] = (int32_t)i;
            todo = false;
          }
          if (tid == leader) base[e0] += __builtin_popcountll(same);
          // wave-synchronous: the next iteration's reads of base[] follow this write in program order
          __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        }
      }
    }
  }
  // ---- 4. padding, block -> expert map, unused tail (trailing blocks name expert 0) -------------------------
  for (int e = b; e < E; e += B) {
    for (int32_t s2 = start[e] + total[e] + tid; s2 < start[e + 1]; s2 += T) sorted_ids[s2] = (int32_t)n;
    for (int32_t s2 = start[e] + tid * tile_m; s2 < start[e + 1]; s2 += T * tile_m) expert_ids[s2 / tile_m] = e;
  }
  const int32_t used = start[E];
  for (int64_t i = used + (int64_t)b * T + tid; i < max_slots; i += (int64_t)B * T) sorted_ids[i] = (int32_t)n;
  for (int64_t blk = used / tile_m + (int64_t)b * T + tid; blk < max_slots / tile_m; blk += (int64_t)B * T)
    expert_ids[blk] = 0;
}

// ================================================================================================
// Split-K reduction: C = sum of the fp32 partial products (analogue of the second pass of
// matmul_split_k_kernel, test/kernels/matmul.py:103-140)
// ================================================================================================
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, int splits,
                                                            int64_t M, int64_t N, void* C, int64_t ldc,
                                                            int c_dtype, int accumulate) {
  const int64_t n4 = (N + 3) / 4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * n4) return;
  const int64_t m = i / n4, n = (i % n4) * 4;
  const int cnt = N - n >= 4 ? 4 : (int)(N - n);
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  for (int p = 0; p < splits; ++p) {   // fixed order: results do not depend on scheduling
    const float* src = part + ((int64_t)p * M + m) * N + n;
    if (cnt == 4 && (N & 3) == 0) {
      const v4f t = *(const v4f*)src;
      s[0] += t.x; s[1] += t.y; s[2] += t.z; s[3] += t.w;
    } else {
      for (int e = 0; e < cnt; ++e) s[e] += src[e];
    }
  }
  if (c_dtype == MX_F32) {
    float* c = (float*)C + m * ldc + n;
    for (int e = 0; e < cnt; ++e) c[e] = accumulate ? c[e] + s[e] : s[e];
  } else {
    uint16_t* c = (uint16_t*)C + m * ldc + n;
    for (int e = 0; e < cnt; ++e) c[e] = f32_to_bf16(accumulate ? bf16_to_f32(c[e]) + s[e] : s[e]);
  }
}

}  // namespace

int launch_quantize(const QuantArgs& q, hipStream_t stream) {
  const int64_t units = q.rows * (q.Kpad / 32) * (32 / kQuantEpl);
  if (units <= 0) return MX_OK;
  const int64_t blocks = (units + 256 * kQuantUnroll - 1) / (256 * kQuantUnroll);
  if (blocks > 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "quantize: tensor too large");
  hipLaunchKernelGGL(quantize_kernel<kQuantEpl>, dim3((unsigned)blocks), dim3(256), 0, stream, q);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "quantize_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

int launch_pack_scales_pair(const PackArgs* a, const PackArgs* b, hipStream_t stream) {
  PackPair pp = {};
  int64_t blocks[2] = {0, 0};
  const PackArgs* ops[2] = {a, b};
  int n = 0;
  for (int i = 0; i < 2; ++i) {
    const PackArgs* p = ops[i];
    if (!p || p->rows <= 0 || p->K <= 0 || p->batch <= 0) continue;
    pp.p[n] = *p;
    blocks[n] = ((p->rows + 63) / 64) * ((packed_scale_quads(p->K) + 3) / 4) * p->batch;
    ++n;
  }
  if (n == 0) return MX_OK;
  const int64_t total = blocks[0] + blocks[1];
  if (total > 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "pack_scales: tensor too large");
  pp.blocks0 = (int32_t)blocks[0];
  hipLaunchKernelGGL(pack_scales_kernel, dim3((unsigned)total), dim3(256), 0, stream, pp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "pack_scales_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

int launch_pack_scales_list(const PackArgs* list, int n, hipStream_t stream) {
  for (int i0 = 0; i0 < n; i0 += kPackListMax) {
    PackList pl = {};
    int64_t total = 0;
    for (int i = i0; i < n && i < i0 + kPackListMax; ++i) {
      const PackArgs& p = list[i];
      if (p.rows <= 0 || p.K <= 0 || p.batch <= 0) continue;
      if (p.layout != MX_SCALE_2D || p.batch != 1 || p.gather_ids)
        return set_error(MX_ERR_INVALID, "pack_scales list: plain 2-D scale tensors only");
      pl.p[pl.n] = PackEntry{p.src, p.dst, p.rows, p.K, p.s_row, p.s_kb, p.target};
      pl.first_block[pl.n] = (int32_t)total;
      total += ((p.rows + 63) / 64) * ((packed_scale_quads(p.K) + 3) / 4) * p.batch;
      if (total > 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "pack_scales: tensors too large");
      ++pl.n;
    }
    if (pl.n == 0) continue;
    pl.first_block[pl.n] = (int32_t)total;
    hipLaunchKernelGGL(pack_scales_list_kernel, dim3((unsigned)total), dim3(256), 0, stream, pl);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "pack_scales_list_kernel launch: %s", hipGetErrorString(e));
  }
  return MX_OK;
}

int launch_pack_scales(const PackArgs& p, hipStream_t stream) {
  return launch_pack_scales_pair(&p, nullptr, stream);
}

int launch_splitk_reduce(const float* partials, int splits, int64_t M, int64_t N, void* C, int64_t ldc,
                         int c_dtype, int accumulate, hipStream_t stream) {
  const int64_t threads = M * ((N + 3) / 4);
  if (threads <= 0) return MX_OK;
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, partials,
                     splits, M, N, C, ldc, c_dtype, accumulate);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "splitk_reduce_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

// chunks (= workgroups) the ids are cut into: about 1024 ids each, at most 256 chunks unless a chunk would then
// exceed what the u16 prefixes of the placement hold
void moe_align_plan(int64_t num_ids, int64_t& chunk, int64_t& blocks) {
  chunk = (num_ids + 255) / 256;
  if (chunk < 1024) chunk = 1024;
  if (chunk > kAlignMaxChunk) chunk = kAlignMaxChunk;
  blocks = num_ids > 0 ? (num_ids + chunk - 1) / chunk : 1;
}

int64_t moe_align_workspace_bytes(int64_t num_ids, int32_t num_experts) {
  int64_t chunk, blocks;
  moe_align_plan(num_ids, chunk, blocks);
  return blocks > 1 ? blocks * num_experts * (int64_t)sizeof(int32_t) : 0;
}

int launch_moe_align(const int32_t* topk_ids, int64_t num_ids, int32_t num_experts, int32_t tile_m,
                     int32_t* sorted_token_ids, int32_t* sorted_expert_ids, int32_t* num_slots_out,
                     int64_t max_slots, int32_t* counts, hipStream_t stream) {
  int64_t chunk, blocks;
  moe_align_plan(num_ids, chunk, blocks);
  const bool seg = num_experts <= kAlignSegExperts;
  const size_t lds = (size_t)(3 * num_experts + 1 + kAlignThreads) * sizeof(int32_t) +
                     (seg ? (size_t)num_experts * (kAlignThreads + 2) * sizeof(uint16_t) : 0);
  if (lds > 150 * 1024) return set_error(MX_ERR_SHAPE, "moe_align: too many experts (%d)", num_experts);
  if (blocks > 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "moe_align: too many ids");
  static int attr_done = 0;   // benign race: the attribute call is idempotent
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)moe_place_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       160 * 1024);
    if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "hipFuncSetAttribute(moe_align): %s", hipGetErrorString(e));
    attr_done = 1;
  }
  if (blocks > 1) {
    hipLaunchKernelGGL(moe_hist_kernel, dim3((unsigned)blocks), dim3(kAlignThreads), (size_t)num_experts * sizeof(int32_t),
                       stream, topk_ids, num_ids, num_experts, chunk, counts);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "moe_hist_kernel launch: %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(moe_place_kernel, dim3((unsigned)blocks), dim3(kAlignThreads), lds, stream, topk_ids, num_ids,
                     num_experts, tile_m, chunk, counts, sorted_token_ids, sorted_expert_ids, num_slots_out, max_slots);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "moe_place_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

}  // namespace mx
