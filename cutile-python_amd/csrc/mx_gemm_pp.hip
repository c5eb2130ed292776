// Persistent ping-pong block-scaled GEMM for large problems (gfx950): 256 x 256 tile, 8 waves.
//
// Same math, operand layouts and LDS swizzle as the kernel in mx_gemm_mfma.hip; what differs is the
// schedule.  The 8 waves form two teams of four (one wave of each team per SIMD): team 0 owns rows
// 0-127 of the tile, team 1 rows 128-255; wave (team, wn) computes the 128 x 64 block at columns
// 64 wn.  Every K stage of a wave is split into
//   a MEMORY phase: LDS-DMA issue for stage s + 2, LDS reads of the B fragments and the first A
//                   tiles of stage s;
//   an MFMA phase:  32 (64 for FP4) back-to-back MFMAs from registers, with the reads of the other
//                   remaining A tiles slotted in 8 or 16 MFMAs ahead of their use.
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
//
// Persistence: a workgroup walks a list of tiles.  The stage pipeline runs straight across tile
// boundaries (the last two stages of a tile prefetch the first two of the next one), and the output
// of a finished tile is converted and stored inside the first memory phase of the next tile, i.e.
// while the other team is in an MFMA phase, so neither the pipeline fill nor the epilogue idles the
// matrix pipe.  A workgroup is given more than one tile only when a tile has at least two stages and
// a whole number of K-quads (K a multiple of 512).
#include <stdlib.h>

#include <type_traits>

#include "mx_gemm_pp.h"

namespace mx {
namespace {

// Output of a tile that touches the matrix edge, accumulates into C or has an unaligned C: every
// element checked.  Deliberately not inlined (the accumulators are passed by value) so that its address
// arithmetic and branches stay out of the register allocation of the main loop.
struct AccTile {
  v4f v[8][4];
};

template <typename OutT>
__device__ __attribute__((noinline)) void write_tile_checked(AccTile t, OutT* Cp, int64_t ldc, int M, int N,
                                                             int mw, int nw, bool accumulate,
                                                             bool vec_ok) {
  // mw / nw: row of the lane in tile (0, j) / first column of the lane in tile (i, 0); tile (i, j) starts
  // bperm_tile_off(j) columns further
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = mw + 16 * i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = nw + bperm_tile_off(j);
      if (n >= N) continue;
      store4<OutT>(Cp + (int64_t)m * ldc + n, t.v[i][j], accumulate, N - n, vec_ok);
    }
  }
}

// KTAIL: K is not a whole number of stages (or there is a single stage): the 16-byte chunks beyond the end of K are
// masked lane by lane at issue time.  Without it the loads take their precomputed offsets as they are, which keeps a
// compare and a select per DMA instruction out of the memory phase.
template <class C, typename OutT, bool GROUPED, int TEAM, bool KTAIL>
__device__ __forceinline__ void pp_body(const GemmArgs& g, lds_u8* const smem, const int wn,
                                        const int lane, const TileWalk& walk) {
  using P = PP<C>;
  constexpr int AL = P::AL, BL = P::BL;
  // A tiles (of 8) whose fragments are read in the memory phase; the others are read inside the MFMA phase,
  // 8 MFMAs ahead of their use.  Two measured best (four: 1.5 % slower on MXFP8, 5 % on the grouped
  // variant: the longer memory phase costs more than the later reads)
  constexpr int EARLY = 2;
  const int r = lane & 15, gq = lane >> 4;
  constexpr int wm0 = TEAM * 128;
  const int wn0 = wn * 64;

  const int Kb_a = g.K * C::A_EB / 8, Kb_b = g.K * C::B_EB / 8;
  const int ksteps = (g.K + 127) / 128;
  const int nstages = (ksteps + C::KSUB - 1) / C::KSUB;
  const int KQ = (ksteps + 3) / 4;
  const int a_groups = (g.M + 63) / 64, b_groups = (g.N + 63) / 64;
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.A, (uint32_t)(g.a_rows * g.lda));

  // ---- load context: where the DMA and scale loads of the tile being FETCHED point --------------------
  // A: instruction q of the wave covers tile rows wm0 + (4 q + wn) * A_RPI ...; B (team 1 only):
  // rows wn0 + q * B_RPI ....  A: the swizzled byte column of instruction q is col0 ^ (4 q % CPR) * 16.
  uint32_t a_voff[AL], b_voff[TEAM ? BL : 1];
  const int a_row0 = wm0 + wn * P::A_RPI + lane / C::A_CPR;
  const int a_col0 = ((lane % C::A_CPR) ^ swz<C::A_CPR>(a_row0)) * 16;
  const int b_row0 = wn0 + lane / C::B_CPR;
  // swizzled byte column of DMA instruction q (rows b_row0 + q * B_RPI ...)
  auto b_col = [&](int q) { return ((lane % C::B_CPR) ^ swz_bperm<C::B_CPR>(lane / C::B_CPR + q * P::B_RPI)) * 16; };
  __amdgpu_buffer_rsrc_t rsB;
  // ---- scales (native layout, mx_common.h): 16 bytes per (64-row group, K-quad, lane), dword t = K-step t of the
  // quad, byte = 16-row tile of the group (B: in the bperm_row order of the fragments).  A K-quad needs the team's
  // two A groups and the wave's one B group: three 16-byte loads (1 KiB contiguous per wave) through buffer
  // descriptors, the (group, quad) part of the address in the scalar offset.
  // as / bs _cur, _nxt: byte offset of (group, K-quad 0) for the tile being computed / being fetched.
  int as_cur[2], bs_cur, as_nxt[2], bs_nxt;
  const __amdgpu_buffer_rsrc_t rsAs = make_rsrc(g.As, (uint32_t)(packed_scale_dwords(g.M, g.K) * 4));
  const __amdgpu_buffer_rsrc_t rsBs =
      make_rsrc(g.Bs, (uint32_t)((GROUPED ? (int64_t)(g.num_experts - 1) * g.bs_expert_stride * 4 : 0) +
                                 packed_scale_dwords(g.N, g.K) * 4));
  const int sc_voff = lane * 16;
  constexpr int NSC = 3;           // scale load instructions per K-quad
  v4i sa[2], sb;
  auto load_scales = [&](const int* as_off, int bs_off, int Qn) {
#pragma unroll
    for (int u = 0; u < 2; ++u) sa[u] = __builtin_amdgcn_raw_buffer_load_b128(rsAs, sc_voff, as_off[u] + Qn * 1024, 0);
    sb = __builtin_amdgcn_raw_buffer_load_b128(rsBs, sc_voff, bs_off + Qn * 1024, 0);
  };
  bool fetch_valid = true;   // false once the walk has no further tile: loads become zero-fill no-ops
  // grouped: none of this team's 128 slots of the tile holds a routed row (every slot is looked at: two per lane,
  // then a vote, so a sentinel in front of valid ids does not hide them).  Such a half has nothing to multiply:
  // its fragment reads and MFMAs are skipped.
  bool skip_cur = false, skip_nxt = false;
  auto set_fetch_tile = [&](int lid) {
    fetch_valid = lid < walk.end;
    int m0 = 0, n0 = 0;
    if (fetch_valid) walk.origin(lid, m0, n0);
    if constexpr (GROUPED) {
      skip_nxt = false;
      if (fetch_valid) {
        bool any = false;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int m = m0 + wm0 + 64 * u + lane;
          const int id = m < g.M ? g.sorted_token_ids[m] : -1;
          any = any || (id >= 0 && id < g.num_valid_ids);
        }
        skip_nxt = __builtin_amdgcn_ballot_w64(any) == 0;
      }
    }
    int expert = 0;
    if constexpr (GROUPED) {
      // an id outside [0, experts) would move the descriptor's base past W, where the range check no longer helps
      expert = g.sorted_expert_ids[m0 / g.tile_m];
      expert = expert < 0 ? 0 : (expert >= g.num_experts ? g.num_experts - 1 : expert);
    }
    const uint8_t* Bbase = g.B + (GROUPED ? (int64_t)expert * g.b_expert_stride : 0);
    rsB = make_rsrc(Bbase, (uint32_t)((int64_t)g.N * g.ldb));
#pragma unroll
    for (int q = 0; q < AL; ++q) {
      int64_t grow = m0 + a_row0 + q * 4 * P::A_RPI;
      bool ok = fetch_valid && grow < g.M;
      if constexpr (GROUPED) {
        const int id = ok ? g.sorted_token_ids[grow] : 0x7FFFFFFF;
        ok = ok && id >= 0 && id < g.num_valid_ids;
        grow = id / g.replicas;
      }
      a_voff[q] = ok ? (uint32_t)(grow * g.lda + a_col0) : kOobOffset;
    }
    if constexpr (TEAM == 1) {
#pragma unroll
      for (int q = 0; q < BL; ++q) {
        const int col = b_col(q);
        const int64_t grow = n0 + b_row0 + q * P::B_RPI;
        b_voff[q] = (fetch_valid && grow < g.N) ? (uint32_t)(grow * g.ldb + col) : kOobOffset;
      }
    }
    // a tile that overhangs the matrix reuses the last scale group (its rows are discarded anyway)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int grp = (m0 + wm0) / 64 + u;
      as_nxt[u] = (grp < a_groups ? grp : a_groups - 1) * KQ * 1024;
    }
    const int grp = (n0 + wn0) / 64;
    bs_nxt = (GROUPED ? (int)(expert * (g.bs_expert_stride * 4)) : 0) +
             (grp < b_groups ? grp : b_groups - 1) * KQ * 1024;
  };
  // local stage sl of the fetch tile into A buffer abuf / B buffer bbuf; a stage at or beyond nstages
  // and the 16-byte chunks beyond the end of K read nothing and zero-fill their LDS bytes
  // (out-of-range buffer offset)
  auto issue_a = [&](int sl, int abuf) {
    lds_u8* const base = smem + abuf * C::A_STAGE + wm0 * C::A_RB + wn * 1024;
    const int ka = sl * C::A_RB;
    const int klim = sl < nstages ? Kb_a - ka : 0;   // bytes of this stage's rows that exist
#pragma unroll
    for (int q = 0; q < AL; ++q) {
      // (without a K tail a stage at or beyond nstages is only ever requested once the walk has no further tile, and
      // then every offset is out of range already)
      const uint32_t v = (KTAIL && a_col0 >= klim) ? kOobOffset : a_voff[q];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_void*)(base + q * 4096), 16, v, ka, 0, 0);
    }
  };
  auto issue_b = [&](int sl, int bbuf, int q0 = 0, int q1 = P::BL) {   // DMA instructions q0 .. q1 - 1
    if constexpr (TEAM == 1) {
      lds_u8* const base = smem + P::B_BASE + bbuf * C::B_STAGE + wn0 * C::B_RB;
      const int kb = sl * C::B_RB;
      const int klim = sl < nstages ? Kb_b - kb : 0;
#pragma unroll
      for (int q = q0; q < q1; ++q) {
        const int col = b_col(q);
        const uint32_t v = (KTAIL && col >= klim) ? kOobOffset : b_voff[q];
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_void*)(base + q * 1024), 16, v, kb, 0, 0);
      }
    }
  };

  v4f acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  const int swa = swz<C::A_CPR>(r), swb = swz<C::B_CPR>(r);
  constexpr int SPQ = 4 / C::KSUB;   // stages per K-quad

  // ---- output of a finished tile: lane (c, g) of tile (i, j) holds row 16 i + c, columns
  // 32 (j / 2) + 8 g + 4 (j % 2) .. + 3 (see bperm_tile_off); the accumulators are cleared for the next tile ------------------------------------
  OutT* const Cp = (OutT*)g.C;
  const bool vec_ok = (g.ldc % 4 == 0) && (((uintptr_t)g.C) % 16 == 0);
  // the lane's 8 consecutive outputs of a tile pair as 16-byte stores: every row start 16-byte aligned
  const bool vec8_ok = ((g.ldc * (int64_t)sizeof(OutT)) % 16 == 0) && (((uintptr_t)g.C) % 16 == 0);
  const bool accumulate = g.accumulate != 0;
  int eid[2] = {-1, -1};
  auto write_tile = [&](int m0, int n0) {
    if constexpr (!GROUPED) {
      // interior tile, plain store: one address per lane, everything else immediate offsets
      if (m0 + 256 <= g.M && n0 + 256 <= g.N && vec8_ok && !accumulate) {
        OutT* p = Cp + (int64_t)(m0 + wm0 + r) * g.ldc + (n0 + wn0 + 8 * gq);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
          for (int jp = 0; jp < 2; ++jp) {
            store8_full<OutT>(p + 32 * jp, acc[i][2 * jp], acc[i][2 * jp + 1]);
            acc[i][2 * jp] = (v4f){0.f, 0.f, 0.f, 0.f};
            acc[i][2 * jp + 1] = (v4f){0.f, 0.f, 0.f, 0.f};
          }
          p += 16 * g.ldc;
        }
        return;
      }
      AccTile t;
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          t.v[i][j] = acc[i][j];
          acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
        }
      write_tile_checked<OutT>(t, Cp, g.ldc, g.M, g.N, m0 + wm0 + r, n0 + wn0 + 8 * gq, accumulate, vec_ok);
      return;
    }
    // grouped: row 16 i + c of the team's half goes to row `id` of C, where id is the routed-slot index
    // that lane 16 (i % 4) + c of eid[i / 4] has held since the tile began (no load latency here)
    const bool cols_in = n0 + 256 <= g.N && vec8_ok && !accumulate;   // uniform
    float ewt[2] = {1.f, 1.f};
    if (g.topk_weights) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
        if (eid[u] >= 0 && eid[u] < g.num_valid_ids) ewt[u] = g.topk_weights[eid[u]];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int src = (16 * (i & 3) + r) * 4;
      const int id = __builtin_amdgcn_ds_bpermute(src, eid[i >> 2]);
      const bool ok = id >= 0 && id < g.num_valid_ids;
      float w = 1.f;
      if (g.topk_weights) w = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src, __builtin_bit_cast(int, ewt[i >> 2])));
      OutT* const p = Cp + (int64_t)id * g.ldc + (n0 + wn0 + 8 * gq);
      if (cols_in) {
        if (ok) {
#pragma unroll
          for (int jp = 0; jp < 2; ++jp) store8_full<OutT>(p + 32 * jp, acc[i][2 * jp] * w, acc[i][2 * jp + 1] * w);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = n0 + wn0 + 8 * gq + bperm_tile_off(j);
          if (ok && n < g.N)
            store4<OutT>(p + bperm_tile_off(j), acc[i][j] * w, accumulate, g.N - n, vec_ok);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
    }
  };
  // grouped: the routed-slot ids of the team's 128 rows of the tile at m0, two per lane
  auto load_row_ids = [&](int m0) {
    if constexpr (GROUPED) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int m = m0 + wm0 + 64 * u + lane;
        eid[u] = m < g.M ? g.sorted_token_ids[m] : -1;
      }
    }
  };

  // ---- prologue: stages 0 and 1 of the first tile, scales of its K-quad 0 ---------------------------------
  int lid = walk.first;          // tile being computed
  set_fetch_tile(lid);
  {
    int fm0, fn0;
    walk.origin(lid, fm0, fn0);
    load_row_ids(fm0);
  }
  issue_a(0, 0);
  issue_b(0, 0);
  issue_a(1, 1);
  issue_b(1, 1);
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
    if constexpr (t0 == 0) {
      // Scales of this K-quad, first in the queue of this memory phase: they have the whole phase to arrive, and
      // the MFMA phase holds no vector-memory instruction at all.  (Requested a stage ahead, stage by stage, in
      // 4-byte loads, they arrive no earlier in effect: what they cost is their share of the address unit, which
      // three 16-byte loads per quad keep smallest.)
      load_scales(as_cur, bs_cur, Q);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (t0 == 0) {
      if (s == 0 && lid != walk.first) {
        // the previous tile's output leaves while the other team is in its MFMA phase
        // (the tile index passes through an opaque move: otherwise the compiler computes the eight row
        // pointers of the stores when the tile begins and keeps them in registers through all its stages)
        int plid = lid - walk.step;
        asm volatile("" : "+s"(plid));
        int pm0, pn0;
        walk.origin(plid, pm0, pn0);
        write_tile(pm0, pn0);
        if constexpr (GROUPED) {
          walk.origin(lid, pm0, pn0);
          load_row_ids(pm0);
        }
      }
    }
    // from stage nstages - 2 on, the loads run ahead into the next tile of the walk
    if (s + 2 == nstages) set_fetch_tile(lid + walk.step);
    const bool wrapped = s + 2 >= nstages;
    const int sl = wrapped ? s + 2 - nstages : s + 2;   // local stage the loads fetch
    const int sl_eff = (wrapped && (!fetch_valid || nstages < 2)) ? nstages : sl;
    lds_u8* const atile = smem + abuf * C::A_STAGE + (wm0 + r) * C::A_RB;
    lds_u8* const btile = smem + P::B_BASE + bbuf * C::B_STAGE + (wn0 + bperm_lane_off(r)) * C::B_RB;
    issue_a(sl_eff, abuf2);
    v8i bf[C::KSUB][4], af[C::KSUB][8];
    if (!(GROUPED && skip_cur)) {
      // B tiles 0, 1 (rows 0 .. 31 of the wave's 64), then tiles 2, 3, then the early A tiles: LDS returns reads in
      // order, so the DMA that refills the first half of the B rows can go as soon as the first group is back
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int kk = 0; kk < C::KSUB; ++kk)
#pragma unroll
          for (int j = 2 * h; j < 2 * h + 2; ++j) bf[kk][j] = load_frag<C::B_RB, C::B_EB>(btile, bperm_tile_off(j), kk, gq, swb);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int kk = 0; kk < C::KSUB; ++kk)
#pragma unroll
        for (int i = 0; i < EARLY; ++i) af[kk][i] = load_frag<C::A_RB, C::A_EB>(atile, 16 * i, kk, gq, swa);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (TEAM == 1) {
      // the B buffer of this stage is free once this wave's own reads have returned
      constexpr int NBH = 2 * C::KSUB * (C::B_EB == 8 ? 2 : 1);       // LDS reads of two B tiles
      constexpr int NAE = EARLY * C::KSUB * (C::A_EB == 8 ? 2 : 1);   // LDS reads of the early A tiles
      asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(NBH + NAE) : "memory");
      __builtin_amdgcn_sched_barrier(0);
      issue_b(sl_eff, bbuf, 0, BL / 2);
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(NAE) : "memory");
      __builtin_amdgcn_sched_barrier(0);
      issue_b(sl_eff, bbuf, BL / 2, BL);
      // everything older than this phase's loads has landed: A and B of stage s + 1 (the scale loads issued
      // at the start of this phase are younger than those and may stay in flight; the MFMA phase waits for them)
      constexpr int younger = (t0 == 0) ? NSC : 0;
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(AL + BL + younger));
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // fragments are in registers
    __builtin_amdgcn_sched_barrier(0);
    // =============================== MFMA phase ====================================================
    __builtin_amdgcn_s_setprio(1);
    auto read_pair = [&](int i0) {
#pragma unroll
      for (int kk = 0; kk < C::KSUB; ++kk)
#pragma unroll
        for (int i = i0; i < i0 + 2; ++i) {
          af[kk][i] = load_frag<C::A_RB, C::A_EB>(atile, 16 * i, kk, gq, swa);
        }
      __builtin_amdgcn_sched_barrier(0);
    };
    auto mfma_pair = [&](int i0, int n = 2) {   // row tiles i0 .. i0 + n - 1
#pragma unroll
      for (int kk = 0; kk < C::KSUB; ++kk) {
#pragma unroll
        for (int i = i0; i < i0 + n; ++i) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[i][j] = mfma_scaled<C::BF, C::AF>(bf[kk][j], af[kk][i], acc[i][j], j, sb[t0 + kk], i % 4,
                                                  sa[i / 4][t0 + kk]);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // A tiles below EARLY were read in the memory phase; the rest is read EARLY * 4 MFMAs ahead of use
    if (!(GROUPED && skip_cur)) {
#pragma unroll
      for (int ip = 0; ip < 8; ip += 2) {
        if (ip == 0) {
          // the phase opens with MFMAs, not with LDS read issue: the matrix pipe restarts that much sooner after the
          // hand-over, and the reads issue while the first MFMAs run
          mfma_pair(0, 1);
          read_pair(EARLY);
          mfma_pair(1, 1);
          continue;
        }
        if (ip + EARLY < 8) read_pair(ip + EARLY);
        mfma_pair(ip);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (TEAM == 0) {
      // A of stage s + 1 (issued one stage ago) must have landed; A of stage s + 2 may stay in flight
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(AL));
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    abuf = abuf == 2 ? 0 : abuf + 1;
    abuf2 = abuf2 == 2 ? 0 : abuf2 + 1;
    bbuf ^= 1;
  };
  for (; lid < walk.end; lid += walk.step) {
    skip_cur = skip_nxt;
    as_cur[0] = as_nxt[0];
    as_cur[1] = as_nxt[1];
    bs_cur = bs_nxt;
    for (Q = 0; Q < KQ; ++Q) {
      stage(std::integral_constant<int, 0>{});
      if constexpr (C::KSUB == 1) stage(std::integral_constant<int, 1>{});
      stage(std::integral_constant<int, 2>{});
      if constexpr (C::KSUB == 1) stage(std::integral_constant<int, 3>{});
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // trailing zero-fill DMA has left the queue
  __builtin_amdgcn_sched_barrier(0);
  {
    int pm0, pn0;
    walk.origin(lid - walk.step, pm0, pn0);
    write_tile(pm0, pn0);
  }
  if constexpr (TEAM == 0) asm volatile("s_barrier" ::: "memory");   // pairs with team 1's extra barrier
}

template <class C, typename OutT, bool GROUPED>
__global__ __launch_bounds__(512) void gemm_pp_kernel(const GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_generic[];
  lds_u8* const smem = (lds_u8*)smem_generic;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  const TileWalk walk = make_tile_walk(g.M, g.N);
  if (walk.first >= walk.end) return;   // cannot happen with the grids the launcher picks
  const int ksteps = (g.K + 127) / 128;
  // (uniform.  The MXFP4 instance keeps the one masked body: a second, unmasked one measured no faster on it.)
  const bool ktail = C::KSUB != 1 || g.K % 128 != 0 || ksteps < 2;
  if (ktail) {
    if (wave < 4)
      pp_body<C, OutT, GROUPED, 0, true>(g, smem, wave, lane, walk);
    else
      pp_body<C, OutT, GROUPED, 1, true>(g, smem, wave - 4, lane, walk);
  } else if constexpr (C::KSUB == 1) {
    if (wave < 4)
      pp_body<C, OutT, GROUPED, 0, false>(g, smem, wave, lane, walk);
    else
      pp_body<C, OutT, GROUPED, 1, false>(g, smem, wave - 4, lane, walk);
  }
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
  const int64_t grid = pp_grid(g.M, g.N, g.K, C::KSUB);
  if (grid <= 0) return MX_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), PP<C>::LDS_BYTES, stream, g);
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
