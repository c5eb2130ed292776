// Persistent block-scaled GEMM with four waves per workgroup (gfx950): 256 x 256 tile, every wave owns a
// 128 x 128 quarter, v_mfma_scale_f32_32x32x64_f8f6f4, 8-bit element formats.
//
// Why a second large-tile kernel: in the eight-wave ping-pong kernels (mx_gemm_pp.hip) a wave's block is 128 x 64,
// so a 128-element K stage costs the workgroup 8 x (128 + 64) = 1536 fragment rows of LDS reads; with 128 x 128
// per wave it is 4 x 256 = 1024, a third less.  The 256 accumulator registers of such a wave only fit with one
// wave per SIMD (512 registers, the accumulators in the AGPR half), so there is no second wave to hide latency
// behind: the wave software-pipelines itself.
//
// Pipeline.  The K walk is cut into half-stages of 64 elements (one 32x32x64 instruction deep).  LDS holds a ring of
// five half-stage buffers (32 KiB each: 256 A rows and 256 B rows of 64 bytes, 16-byte chunks XOR-swizzled by row).
// In half-stage G a wave
//   * issues its 16 matrix instructions from the fragments of half-stage G, which are already in registers,
//   * reads the fragments of half-stage G + 1 from LDS into the other register set (first 8 instruction slots),
//   * in even G, issues its share of the LDS-DMA loads of half-stages G + 4 and G + 5 (the two 64-byte halves of
//     the same 128-byte pieces of the operand rows, back to back so that the second half finds its cache line),
//   * waits for its own loads up to half-stage G + 2 (everything but the latest batch) and for its LDS reads, and
//     meets the other three waves at the one barrier of the half-stage, placed a few instructions before the end
//     so that the matrix pipe keeps running while the waves gather.
// A load therefore has three to four half-stages (about 1.5 us) to land.  The ring runs across tile boundaries:
// the loads of the next tile's first half-stages are in flight while a tile's output is converted and stored.
//
// Operand layout of the instruction, row permutation of the B fragment and scale addressing are those of
// mx_gemm_pp32.hip: lane (r, g) = (lane % 32, lane / 32) holds bytes 16 g .. and 32 + 16 g .. of the row's
// 64-byte half-stage; the scale of K block kb is read from lane group kb; operand row 8 a + 4 h + c of the B
// fragment is B row 16 h + 4 a + c, which gives lane (c, h) the 16 consecutive outputs 16 h .. of row c.
#include <stdlib.h>

#include <type_traits>

#include "mx_gemm_pp.h"

namespace mx {
namespace {

typedef float v16f_t __attribute__((ext_vector_type(16)));

constexpr int kRing = 5;                 // half-stage buffers
constexpr int kBuf = 32768;              // bytes of one: A [256][64], then B [256][64]
constexpr int kBufB = 16384;             // offset of the B rows
constexpr int kLds = kRing * kBuf;
constexpr int kBatch = 16;               // DMA instructions a wave issues per even half-stage

__device__ inline int w4_brow(int i) { return 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3); }
// swizzle terms of 64-byte rows (4 chunks): rows that share row % 4 share the bank quarter and must differ here
__device__ inline int w4_swz_a(int row) { return (row >> 2) & 3; }                          // rows c = 0 .. 15 of a read
__device__ inline int w4_swz_b(int row) { return ((row >> 2) & 1) | (((row >> 4) & 1) << 1); }   // rows w4_brow(c)

__device__ inline v4f w4_quad(const v16f_t& v, int q) { return (v4f){v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]}; }

template <int AF, int BF, typename OutT>
__global__ __launch_bounds__(256) void gemm_w4_kernel(const GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_generic[];
  lds_u8* const smem = (lds_u8*)smem_generic;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int m = lane & 31, gh = lane >> 5;
  const int brow = w4_brow(m);

  const TileWalk walk = make_tile_walk(g.M, g.N);
  if (walk.first >= walk.end) return;   // cannot happen with the grids the launcher picks

  const int Kb = g.K;                                   // bytes per operand row
  const int nstages = (g.K + 127) / 128;
  const int H = 2 * nstages;                            // half-stages per tile (the launcher guarantees H >= 6)
  const int KQ = (nstages + 3) / 4;
  const int a_groups = (g.M + 63) / 64, b_groups = (g.N + 63) / 64;
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.A, (uint32_t)(g.a_rows * g.lda));
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(g.B, (uint32_t)((int64_t)g.N * g.ldb));

  // ---- DMA context of the tile being FETCHED: wave w loads rows 64 w .. 64 w + 63 of A and of B, instruction q
  // rows 64 w + 16 q + lane / 4, 16-byte chunk lane % 4 of the 64-byte half row (position XOR swizzle) -----------
  const int ld_row = 64 * wave + (lane >> 2);
  const int a_chunk = ((lane & 3) ^ w4_swz_a(ld_row)) * 16;            // the same for every q
  const int b_chunk0 = ((lane & 3) ^ w4_swz_b(ld_row)) * 16;           // q even
  const int b_chunk1 = ((lane & 3) ^ w4_swz_b(ld_row + 16)) * 16;      // q odd
  uint32_t a_voff[4], b_voff[4];
  int as_cur[2], bs_cur[2], as_nxt[2], bs_nxt[2];   // 16-byte index of (64-row group, K-quad 0, lane 0)
  bool fetch_valid = true;
  auto set_fetch_tile = [&](int lid) {
    fetch_valid = lid < walk.end;
    int m0 = 0, n0 = 0;
    if (fetch_valid) walk.origin(lid, m0, n0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int64_t ar = m0 + ld_row + 16 * q, br = n0 + ld_row + 16 * q;
      a_voff[q] = (fetch_valid && ar < g.M) ? (uint32_t)(ar * g.lda + a_chunk) : kOobOffset;
      b_voff[q] = (fetch_valid && br < g.N) ? (uint32_t)(br * g.ldb + ((q & 1) ? b_chunk1 : b_chunk0)) : kOobOffset;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int ga = (m0 + wm * 128) / 64 + u, gb = (n0 + wn * 128) / 64 + u;
      as_nxt[u] = (ga < a_groups ? ga : a_groups - 1) * KQ * 64;
      bs_nxt[u] = (gb < b_groups ? gb : b_groups - 1) * KQ * 64;
    }
  };
  // instruction (op, q) of half-stage hb of the fetch tile into ring buffer `buf`; hb >= H or chunks beyond the
  // end of K read nothing and zero-fill their LDS bytes (out-of-range buffer offset)
  auto issue_one = [&](bool is_b, int q, int hb, int buf) {
    const int kbyte = hb * 64;
    const int lim = (hb < H && fetch_valid) ? Kb - kbyte : 0;
    if (!is_b) {
      const uint32_t v = a_chunk >= lim ? kOobOffset : a_voff[q];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_void*)(smem + buf * kBuf + (64 * wave + 16 * q) * 64), 16, v,
                                               kbyte, 0, 0);
    } else {
      const int ch = (q & 1) ? b_chunk1 : b_chunk0;
      const uint32_t v = ch >= lim ? kOobOffset : b_voff[q];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_void*)(smem + buf * kBuf + kBufB + (64 * wave + 16 * q) * 64), 16,
                                               v, kbyte, 0, 0);
    }
  };

  // ---- fragment reads: byte offsets of the lane's two chunks inside a buffer, tile 0 of the wave -------------------
  const int a_lo = (wm * 128 + m) * 64 + ((gh ^ w4_swz_a(m)) << 4), a_hi = (wm * 128 + m) * 64 + (((2 + gh) ^ w4_swz_a(m)) << 4);
  const int b_lo = kBufB + (wn * 128 + brow) * 64 + ((gh ^ w4_swz_b(brow)) << 4);
  const int b_hi = kBufB + (wn * 128 + brow) * 64 + (((2 + gh) ^ w4_swz_b(brow)) << 4);
  auto read_frag = [&](int buf, int lo, int hi, int tile) {
    lds_u8* const p = smem + buf * kBuf + tile * 2048;
    const v4i x = *(lds_v4i*)(p + lo);
    const v4i y = *(lds_v4i*)(p + hi);
    return (v8i){x.x, x.y, x.z, x.w, y.x, y.y, y.z, y.w};
  };

  // ---- scales (packed layout of mx_common.h): one 16-byte load brings the dwords of the four 16-row tiles of a
  // 64-row group for lane' = row % 16 + 16 (2 u + kb); the lane keeps the two of its row half.  The loads of the
  // next K-quad are issued at the start of a quad and turned into the operand registers at its end. ----------------
  const v4i* const As4 = (const v4i*)g.As + ((m & 15) + 16 * gh);       // + 32 u
  const v4i* const Bs4 = (const v4i*)g.Bs + ((brow & 15) + 16 * gh);    // + 32 u
  const bool a_up = (m >> 4) != 0, b_up = (brow >> 4) != 0;
  int sa[4][2], sb[4][2];
  v4i ra[2][2], rb[2][2];
  auto load_scales = [&](const int* ai, const int* bi, int Qk) {
#pragma unroll
    for (int gidx = 0; gidx < 2; ++gidx)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        ra[gidx][u] = As4[ai[gidx] + Qk * 64 + 32 * u];
        rb[gidx][u] = Bs4[bi[gidx] + Qk * 64 + 32 * u];
      }
  };
  auto take_scales = [&]() {
#pragma unroll
    for (int gidx = 0; gidx < 2; ++gidx)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        sa[2 * gidx][u] = a_up ? ra[gidx][u].y : ra[gidx][u].x;
        sa[2 * gidx + 1][u] = a_up ? ra[gidx][u].w : ra[gidx][u].z;
        sb[2 * gidx][u] = b_up ? rb[gidx][u].y : rb[gidx][u].x;
        sb[2 * gidx + 1][u] = b_up ? rb[gidx][u].w : rb[gidx][u].z;
      }
  };

  v16f_t acc[4][4];
#pragma unroll
  for (int I = 0; I < 4; ++I)
#pragma unroll
    for (int J = 0; J < 4; ++J)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[I][J][e] = 0.f;

  // ---- output of a finished tile: lane (m, gh) of tile (I, J) holds row 32 I + m, columns 32 J + 16 gh .. + 15 ----
  OutT* const Cp = (OutT*)g.C;
  const bool vec_ok = (g.ldc % 4 == 0) && (((uintptr_t)g.C) % 16 == 0);
  const bool vec8_ok = ((g.ldc * (int64_t)sizeof(OutT)) % 16 == 0) && (((uintptr_t)g.C) % 16 == 0);
  const bool accumulate = g.accumulate != 0;
  auto write_tile = [&](int m0, int n0) {
    const int mrow = m0 + wm * 128 + m, ncol = n0 + wn * 128 + 16 * gh;
    const bool interior = m0 + 256 <= g.M && n0 + 256 <= g.N && vec8_ok && !accumulate;   // uniform
#pragma unroll
    for (int I = 0; I < 4; ++I) {
#pragma unroll
      for (int J = 0; J < 4; ++J) {
        OutT* const p = Cp + (int64_t)(mrow + 32 * I) * g.ldc + (ncol + 32 * J);
        if (interior) {
          store8_full<OutT>(p, w4_quad(acc[I][J], 0), w4_quad(acc[I][J], 1));
          store8_full<OutT>(p + 8, w4_quad(acc[I][J], 2), w4_quad(acc[I][J], 3));
        } else if (mrow + 32 * I < g.M) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int n = ncol + 32 * J + 4 * q;
            if (n < g.N) store4<OutT>(p + 4 * q, w4_quad(acc[I][J], q), accumulate, g.N - n, vec_ok);
          }
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[I][J][e] = 0.f;
      }
    }
  };

  // ---- prologue: half-stages 0 .. 3 of the first tile, scales of its K-quad 0, fragments of half-stage 0 --------
  int lid = walk.first;
  set_fetch_tile(lid);
#pragma unroll
  for (int hb = 0; hb < 4; hb += 2) {
#pragma unroll
    for (int q = 0; q < 4; ++q) { issue_one(false, q, hb, hb); issue_one(false, q, hb + 1, hb + 1); }
#pragma unroll
    for (int q = 0; q < 4; ++q) { issue_one(true, q, hb, hb); issue_one(true, q, hb + 1, hb + 1); }
  }
  load_scales(as_nxt, bs_nxt, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  take_scales();
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  v8i af[2][4], bf[2][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    af[0][t] = read_frag(0, a_lo, a_hi, t);
    bf[0][t] = read_frag(0, b_lo, b_hi, t);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");   // every wave has its fragments of half-stage 0: buffer 0 may be refilled
  __builtin_amdgcn_sched_barrier(0);

  int gbuf = 0;      // ring buffer of the half-stage being computed
  int Q = 0;
  auto half_stage = [&](auto t8c) {
    constexpr int t8 = decltype(t8c)::value;
    constexpr int u = t8 & 1, T = t8 >> 1, cs = t8 & 1, ns = cs ^ 1;
    const int h = Q * 8 + t8;
    if (h >= H) return;
    const int nbuf = gbuf == kRing - 1 ? 0 : gbuf + 1;       // buffer of half-stage h + 1
    if constexpr (t8 == 0) {
      // scales of the next K-quad (quad 0 of the tile being fetched after the last quad), older than this
      // half-stage's batch of DMA loads
      const bool more = Q + 1 < KQ;
      load_scales(more ? as_cur : as_nxt, more ? bs_cur : bs_nxt, more ? Q + 1 : 0);
    }
    int hb = 0, buf4 = 0;
    if constexpr (u == 0) {
      if (h + 4 == H) set_fetch_tile(lid + walk.step);
      hb = h + 4 < H ? h + 4 : h + 4 - H;
      buf4 = gbuf == 0 ? kRing - 1 : gbuf - 1;               // buffer of half-stage h + 4 (h + 5 goes to gbuf)
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int I = k >> 2, J = k & 3;
      acc[I][J] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[cs][J], af[cs][I], acc[I][J], BF, AF, T, sb[J][u], T,
                                                                  sa[I][u]);
      if (k < 4) af[ns][k] = read_frag(nbuf, a_lo, a_hi, k);
      else if (k < 8) bf[ns][k - 4] = read_frag(nbuf, b_lo, b_hi, k - 4);
      if constexpr (u == 0) {
        if (k >= 2 && k < 10) {   // one pair of DMA instructions per slot: the two halves of the same 128-byte pieces
          const int i8 = k - 2;
          issue_one(i8 >= 4, i8 & 3, hb, buf4);
          issue_one(i8 >= 4, i8 & 3, hb + 1, gbuf);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (k == 12) {
        // own loads up to half-stage h + 2 have landed (all but the latest batch), own LDS reads are done
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kBatch) & 0xF0FF);   // ... and lgkmcnt(0)
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (t8 == 7) take_scales();
    gbuf = nbuf;
  };

  for (; lid < walk.end; lid += walk.step) {
#pragma unroll
    for (int u = 0; u < 2; ++u) { as_cur[u] = as_nxt[u]; bs_cur[u] = bs_nxt[u]; }
    for (Q = 0; Q < KQ; ++Q) {
      half_stage(std::integral_constant<int, 0>{});
      half_stage(std::integral_constant<int, 1>{});
      half_stage(std::integral_constant<int, 2>{});
      half_stage(std::integral_constant<int, 3>{});
      half_stage(std::integral_constant<int, 4>{});
      half_stage(std::integral_constant<int, 5>{});
      half_stage(std::integral_constant<int, 6>{});
      half_stage(std::integral_constant<int, 7>{});
      // a K that ends inside the quad: the scales of the next quad / tile are taken here as well
      if ((Q + 1) * 8 > H) take_scales();
    }
    int pm0, pn0;
    walk.origin(lid, pm0, pn0);
    write_tile(pm0, pn0);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // trailing zero-fill DMA has left the queue
}

template <int AF, int BF, typename OutT>
int launch_w4(const GemmArgs& g, hipStream_t stream) {
  auto kern = gemm_w4_kernel<AF, BF, OutT>;
  static int attr_done = 0;   // benign race: the attribute call is idempotent
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess)
      return set_error(MX_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", kLds, hipGetErrorString(e));
    attr_done = 1;
  }
  const int64_t tiles = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
  if (tiles <= 0) return MX_OK;
  const int64_t grid = tiles > num_cus() ? num_cus() : tiles;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), kLds, stream, g);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "gemm_w4_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

}  // namespace

bool gemm_w4_supports(const GemmArgs& g) {
  const bool fmt = (g.a_fmt == MX_E4M3 && g.b_fmt == MX_E4M3) || (g.a_fmt == MX_E5M2 && g.b_fmt == MX_E5M2);
  return fmt && g.sorted_token_ids == nullptr && g.K >= 3 * 128;
}

int launch_gemm_w4(const GemmArgs& g, hipStream_t stream) {
  if (g.c_dtype != MX_F32 && g.c_dtype != MX_BF16)
    return set_error(MX_ERR_DTYPE, "MFMA kernel: output dtype %d not supported", g.c_dtype);
  if (!gemm_w4_supports(g))
    return set_error(MX_ERR_LAYOUT, "the four-wave kernel takes plain (not grouped) products of 8-bit operands with K >= 384");
#define MX_CASE(AFMT, BFMT)                                                                    \
  if (g.a_fmt == AFMT && g.b_fmt == BFMT)                                                      \
    return g.c_dtype == MX_F32 ? launch_w4<AFMT, BFMT, float>(g, stream) : launch_w4<AFMT, BFMT, uint16_t>(g, stream);
  MX_CASE(MX_E4M3, MX_E4M3)
  MX_CASE(MX_E5M2, MX_E5M2)
#undef MX_CASE
  return set_error(MX_ERR_DTYPE, "four-wave kernel: unsupported element format pair (%d, %d)", g.a_fmt, g.b_fmt);
}

}  // namespace mx
