// Ping-pong block-scaled GEMM for large problems (gfx950): 256 x 256 tile, 8 waves.
//
// Same math, operand layouts and LDS swizzle as the kernel in mx_gemm_mfma.hip; what differs is the
// schedule.  The 8 waves form two teams of four (one wave of each team per SIMD): team 0 owns rows
// 0-127 of the tile, team 1 rows 128-255; wave (team, wn) computes the 128 x 64 block at columns
// 64 wn.  Every K stage of a wave is split into
//   a MEMORY phase: LDS-DMA issue for stage s + 2, LDS reads of the B fragments and the first two A
//                   tiles of stage s;
//   an MFMA phase:  32 (64 for FP4) back-to-back MFMAs from registers, with the reads of the other
//                   six A tiles slotted in two tiles ahead of their use.
// One s_barrier ends every phase.  Team 1 runs exactly one phase behind team 0 (it executes one extra
// barrier before its first stage, team 0 one extra after its last), so the two waves of a SIMD are
// never in the same phase: while one waits on LDS, issues DMA or sits in a barrier, the other feeds
// the matrix pipe.
//
// LDS: three A stage buffers (stage s lives in buffer s % 3) and two B stage buffers (s % 2), exactly
// 160 KiB for 128-byte stage rows.  A DMA load is issued two stages ahead of its use.
//   A rows: wave (T, wn) loads a quarter of team T's 128 rows; only team T reads them.
//   B rows: wave (1, wn) loads all 64 rows of column block wn (the rows only waves (0, wn) and (1, wn)
//           read) for stage s + 2 into the buffer of stage s, right after its own reads of stage s;
//           wave (0, wn) read them one phase earlier and will read the new contents three phases
//           later, behind the barrier at which team 1 waits for the loads (vmcnt).
#include <stdlib.h>

#include <type_traits>

#include "mx_gemm_tile.h"

namespace mx {
namespace {

template <class C>
struct PP {
  static_assert(C::BM == 256 && C::BN == 256, "ping-pong kernel is 256 x 256");
  static constexpr int A_BUFS = 3, B_BUFS = 2;
  static constexpr int A_HALF = 128 * C::A_RB;              // bytes of one team's rows in an A buffer
  static constexpr int B_BASE = A_BUFS * C::A_STAGE;
  static constexpr int LDS_BYTES = B_BASE + B_BUFS * C::B_STAGE;
  static constexpr int A_RPI = 64 / C::A_CPR, B_RPI = 64 / C::B_CPR;   // rows per DMA instruction
  static constexpr int AL = 128 / A_RPI / 4;                // A loads per wave and stage
  static constexpr int BL = 64 / B_RPI;                     // B loads per team-1 wave and stage
  static constexpr int SCALE_LOADS = 3;                     // two A groups, one B group
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

template <class C, typename OutT, bool GROUPED, int TEAM>
__device__ __forceinline__ void pp_body(const GemmArgs& g, lds_u8* const smem, const int wn,
                                        const int lane, const int m0, const int n0) {
  using P = PP<C>;
  constexpr int AL = P::AL, BL = P::BL;
  const int r = lane & 15, gq = lane >> 4;
  constexpr int wm0 = TEAM * 128;
  const int wn0 = wn * 64;

  const int Kb_a = g.K * C::A_EB / 8, Kb_b = g.K * C::B_EB / 8;
  const int ksteps = (g.K + 127) / 128;
  const int nstages = (ksteps + C::KSUB - 1) / C::KSUB;
  const int KQ = (ksteps + 3) / 4;

  int expert = 0;
  if constexpr (GROUPED) expert = g.sorted_expert_ids[m0 / g.tile_m];
  const uint8_t* Bbase = g.B + (GROUPED ? (int64_t)expert * g.b_expert_stride : 0);
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.A, (uint32_t)(g.a_rows * g.lda));
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(Bbase, (uint32_t)((int64_t)g.N * g.ldb));

  // ---- DMA work of this lane -----------------------------------------------------------------------
  // A: instruction q of the wave covers tile rows wm0 + (4 q + wn) * A_RPI ...; B (team 1 only):
  // rows wn0 + q * B_RPI ....  The swizzled byte column of instruction q is col0 ^ (4 q % CPR) * 16.
  uint32_t a_voff[AL], b_voff[TEAM ? BL : 1];
  const int a_row0 = wm0 + wn * P::A_RPI + lane / C::A_CPR;
  const int a_col0 = ((lane % C::A_CPR) ^ swz<C::A_CPR>(a_row0)) * 16;
  const int b_row0 = wn0 + lane / C::B_CPR;
  const int b_col0 = ((lane % C::B_CPR) ^ swz<C::B_CPR>(b_row0)) * 16;
#pragma unroll
  for (int q = 0; q < AL; ++q) {
    const int col = a_col0 ^ (((4 * q * 4) % C::A_CPR) << 4);
    int64_t grow = m0 + a_row0 + q * 4 * P::A_RPI;
    bool ok = grow < g.M;
    if constexpr (GROUPED) {
      const int id = ok ? g.sorted_token_ids[grow] : 0x7FFFFFFF;
      ok = ok && id >= 0 && id < g.num_valid_ids;
      grow = id / g.replicas;
    }
    a_voff[q] = ok ? (uint32_t)(grow * g.lda + col) : kOobOffset;
  }
  if constexpr (TEAM == 1) {
#pragma unroll
    for (int q = 0; q < BL; ++q) {
      const int col = b_col0 ^ (((4 * q) % C::B_CPR) << 4);
      const int64_t grow = n0 + b_row0 + q * P::B_RPI;
      b_voff[q] = grow < g.N ? (uint32_t)(grow * g.ldb + col) : kOobOffset;
    }
  }
  // stage s of A into buffer abuf; a stage at or beyond nstages, and the 16-byte chunks beyond the end
  // of K, read nothing and zero-fill their LDS bytes (out-of-range buffer offset)
  auto issue_a = [&](int s, int abuf) {
    lds_u8* const base = smem + abuf * C::A_STAGE + wm0 * C::A_RB + wn * 1024;
    const int ka = s * C::A_RB;
    const int klim = s < nstages ? Kb_a - ka : 0;   // bytes of this stage's rows that exist
#pragma unroll
    for (int q = 0; q < AL; ++q) {
      const int col = a_col0 ^ (((4 * q * 4) % C::A_CPR) << 4);
      const uint32_t v = col >= klim ? kOobOffset : a_voff[q];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_void*)(base + q * 4096), 16, v, ka, 0, 0);
    }
  };
  auto issue_b = [&](int s, int bbuf) {
    if constexpr (TEAM == 1) {
      lds_u8* const base = smem + P::B_BASE + bbuf * C::B_STAGE + wn0 * C::B_RB;
      const int kb = s * C::B_RB;
      const int klim = s < nstages ? Kb_b - kb : 0;
#pragma unroll
      for (int q = 0; q < BL; ++q) {
        const int col = b_col0 ^ (((4 * q) % C::B_CPR) << 4);
        const uint32_t v = col >= klim ? kOobOffset : b_voff[q];
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_void*)(base + q * 1024), 16, v, kb, 0, 0);
      }
    }
  };

  // ---- scales (native layout): one 16-byte load per 64-row group and K-quad ---------------------------
  const v4i* const as_ptr = (const v4i*)g.As + lane;
  const v4i* const bs_ptr =
      (const v4i*)(g.Bs + (GROUPED ? (int64_t)expert * g.bs_expert_stride : 0)) + lane;
  const int a_groups = (g.M + 63) / 64, b_groups = (g.N + 63) / 64;
  int64_t a_sidx[2], b_sidx;   // a tile that overhangs the matrix reuses the last group (rows discarded)
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int grp = (m0 + wm0) / 64 + u;
    a_sidx[u] = (int64_t)(grp < a_groups ? grp : a_groups - 1) * KQ * 64;
  }
  {
    const int grp = (n0 + wn0) / 64;
    b_sidx = (int64_t)(grp < b_groups ? grp : b_groups - 1) * KQ * 64;
  }
  v4i sa[2], sb;

  v4f acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  const int swa = swz<C::A_CPR>(r), swb = swz<C::B_CPR>(r);
  constexpr int SPQ = 4 / C::KSUB;   // stages per K-quad

  // ---- prologue: stages 0 and 1, scales of quad 0 -----------------------------------------------------
  issue_a(0, 0);
  issue_b(0, 0);
  issue_a(1, 1);
  issue_b(1, 1);
#pragma unroll
  for (int u = 0; u < 2; ++u) sa[u] = as_ptr[a_sidx[u]];
  sb = bs_ptr[b_sidx];
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  if constexpr (TEAM == 1) asm volatile("s_barrier" ::: "memory");   // one phase behind team 0
  __builtin_amdgcn_sched_barrier(0);

  int abuf = 0, abuf2 = 2, bbuf = 0;   // buffers of stage s (A, B) and of stage s + 2 (A)
  int Q = 0;
  auto stage = [&](auto t0c) {
    constexpr int t0 = decltype(t0c)::value;
    const int s = Q * SPQ + t0 / C::KSUB;
    if (s >= nstages) return;
    // =============================== memory phase ==================================================
    lds_u8* const atile = smem + abuf * C::A_STAGE + (wm0 + r) * C::A_RB;
    lds_u8* const btile = smem + P::B_BASE + bbuf * C::B_STAGE + (wn0 + r) * C::B_RB;
    issue_a(s + 2, abuf2);
    v8i bf[C::KSUB][4], af[C::KSUB][8];
#pragma unroll
    for (int kk = 0; kk < C::KSUB; ++kk) {
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[kk][j] = load_frag<C::B_RB, C::B_EB>(btile, 16 * j, kk, gq, swb);
#pragma unroll
      for (int i = 0; i < 2; ++i) af[kk][i] = load_frag<C::A_RB, C::A_EB>(atile, 16 * i, kk, gq, swa);
    }
    if constexpr (TEAM == 1) {
      // the B buffer of this stage is free once this wave's own reads have returned
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      issue_b(s + 2, bbuf);
      // everything older than this phase's loads has landed: A and B of stage s + 1
      __builtin_amdgcn_s_waitcnt(0x0F70 | (AL + BL));
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // fragments are in registers
    __builtin_amdgcn_sched_barrier(0);
    // =============================== MFMA phase ====================================================
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int ip = 0; ip < 4; ++ip) {   // pairs of A tiles
      if (ip < 3) {
#pragma unroll
        for (int kk = 0; kk < C::KSUB; ++kk)
#pragma unroll
          for (int i = 2 * ip + 2; i < 2 * ip + 4; ++i)
            af[kk][i] = load_frag<C::A_RB, C::A_EB>(atile, 16 * i, kk, gq, swa);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < C::KSUB; ++kk) {
#pragma unroll
        for (int i = 2 * ip; i < 2 * ip + 2; ++i) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (t0 + kk == 0)
              acc[i][j] = mfma_scaled<C::BF, C::AF, 0>(bf[kk][j], af[kk][i], acc[i][j], sb[j], sa[i / 4][i % 4]);
            else if (t0 + kk == 1)
              acc[i][j] = mfma_scaled<C::BF, C::AF, 1>(bf[kk][j], af[kk][i], acc[i][j], sb[j], sa[i / 4][i % 4]);
            else if (t0 + kk == 2)
              acc[i][j] = mfma_scaled<C::BF, C::AF, 2>(bf[kk][j], af[kk][i], acc[i][j], sb[j], sa[i / 4][i % 4]);
            else
              acc[i][j] = mfma_scaled<C::BF, C::AF, 3>(bf[kk][j], af[kk][i], acc[i][j], sb[j], sa[i / 4][i % 4]);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    constexpr bool last_of_quad = (t0 + C::KSUB == 4);
    if constexpr (last_of_quad) {
      // scales of the next quad; they travel during the barrier and the next memory phase
      const int Qn = Q + 1 < KQ ? Q + 1 : Q;
#pragma unroll
      for (int u = 0; u < 2; ++u) sa[u] = as_ptr[a_sidx[u] + (int64_t)Qn * 64];
      sb = bs_ptr[b_sidx + (int64_t)Qn * 64];
    }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (TEAM == 0) {
      // A of stage s + 1 (issued one stage ago) must have landed; A of stage s + 2 and the scale
      // loads just issued may stay in flight
      __builtin_amdgcn_s_waitcnt(0x0F70 | (AL + (last_of_quad ? P::SCALE_LOADS : 0)));
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    abuf = abuf == 2 ? 0 : abuf + 1;
    abuf2 = abuf2 == 2 ? 0 : abuf2 + 1;
    bbuf ^= 1;
  };
  for (Q = 0; Q < KQ; ++Q) {
    stage(std::integral_constant<int, 0>{});
    if constexpr (C::KSUB == 1) stage(std::integral_constant<int, 1>{});
    stage(std::integral_constant<int, 2>{});
    if constexpr (C::KSUB == 1) stage(std::integral_constant<int, 3>{});
  }
  if constexpr (TEAM == 0) asm volatile("s_barrier" ::: "memory");   // pairs with team 1's extra barrier
  __builtin_amdgcn_s_waitcnt(0x0F70);   // trailing zero-fill DMA has left the queue
  __builtin_amdgcn_sched_barrier(0);

  // ---- epilogue: lane (c, g) of tile (i, j) holds rows 16 i + c, columns 16 j + 4 g .. + 3 -------------
  OutT* const Cp = (OutT*)g.C;
  const bool vec_ok = (g.ldc % 4 == 0) && (((uintptr_t)g.C) % 16 == 0);
  const bool accumulate = g.accumulate != 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = m0 + wm0 + 16 * i + r;
    int64_t orow = m;
    bool ok = m < g.M;
    float w = 1.f;
    if constexpr (GROUPED) {
      const int id = ok ? g.sorted_token_ids[m] : 0x7FFFFFFF;
      ok = ok && id >= 0 && id < g.num_valid_ids;
      orow = id;
      if (ok && g.topk_weights) w = g.topk_weights[id];
    }
    if (!ok) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + wn0 + 16 * j + 4 * gq;
      if (n >= g.N) continue;
      v4f v = acc[i][j];
      if constexpr (GROUPED) v *= w;
      store4<OutT>(Cp + orow * g.ldc + n, v, accumulate, g.N - n, vec_ok);
    }
  }
}

template <class C, typename OutT, bool GROUPED>
__global__ __launch_bounds__(512) void gemm_pp_kernel(const GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_generic[];
  lds_u8* const smem = (lds_u8*)smem_generic;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  // XCD-aware tile order (workgroup ids are dealt round-robin to the 8 XCDs: give each XCD a
  // contiguous range of tiles), then groups of 8 tile rows walked column by column for L2 reuse
  const int tiles_m = (g.M + 255) / 256, tiles_n = (g.N + 255) / 256;
  int tile_m, tile_n;
  {
    const int total = tiles_m * tiles_n;
    const int pid = blockIdx.x;
    const int xcd = pid & 7, loc = pid >> 3, per = total >> 3, rem = total & 7;
    const int lid = xcd * per + (xcd < rem ? xcd : rem) + loc;
    constexpr int GM = 8;
    const int in_group = GM * tiles_n;
    const int gid = lid / in_group, first_m = gid * GM;
    const int gsz = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    const int in = lid % in_group;
    tile_m = first_m + in % gsz;
    tile_n = in / gsz;
  }
  if (wave < 4)
    pp_body<C, OutT, GROUPED, 0>(g, smem, wave, lane, tile_m * 256, tile_n * 256);
  else
    pp_body<C, OutT, GROUPED, 1>(g, smem, wave - 4, lane, tile_m * 256, tile_n * 256);
}

template <class C, typename OutT, bool GROUPED>
int launch_pp(const GemmArgs& g, hipStream_t stream) {
  auto kern = gemm_pp_kernel<C, OutT, GROUPED>;
  static int attr_done = 0;   // benign race: the attribute call is idempotent
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       PP<C>::LDS_BYTES);
    if (e != hipSuccess)
      return set_error(MX_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", PP<C>::LDS_BYTES,
                       hipGetErrorString(e));
    attr_done = 1;
  }
  const int64_t tiles = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
  if (tiles <= 0) return MX_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(512), PP<C>::LDS_BYTES, stream, g);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "gemm_pp_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

}  // namespace

int launch_gemm_pingpong(const GemmArgs& g, hipStream_t stream) {
  if (g.c_dtype != MX_F32 && g.c_dtype != MX_BF16)
    return set_error(MX_ERR_DTYPE, "MFMA kernel: output dtype %d not supported", g.c_dtype);
  const bool grouped = g.sorted_token_ids != nullptr;
#define MX_CASE(AFMT, BFMT)                                                                        \
  if (g.a_fmt == AFMT && g.b_fmt == BFMT) {                                                        \
    using C = Cfg<AFMT, BFMT, 256, 256, 2, 4>;                                                     \
    if (g.c_dtype == MX_F32)                                                                       \
      return grouped ? launch_pp<C, float, true>(g, stream) : launch_pp<C, float, false>(g, stream); \
    return grouped ? launch_pp<C, uint16_t, true>(g, stream) : launch_pp<C, uint16_t, false>(g, stream); \
  }
  MX_CASE(MX_E4M3, MX_E4M3)
  MX_CASE(MX_E5M2, MX_E5M2)
  MX_CASE(MX_E2M1, MX_E2M1)
  MX_CASE(MX_E4M3, MX_E2M1)
#undef MX_CASE
  return set_error(MX_ERR_DTYPE, "MFMA kernel: unsupported element format pair (%d, %d)", g.a_fmt,
                   g.b_fmt);
}

}  // namespace mx
