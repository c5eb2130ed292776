// Block-scaled GEMM on the CDNA4 scaled-MFMA instruction (gfx950).
//
//   C[m, n] (+)= sum_k A[m, k] * As[m, k/32] * B[n, k] * Bs[n, k/32]
//
// A is [M][K] and B is [N][K], both K-contiguous (B is the column-major K x N operand of the
// reference's block_scaled_matmul_kernel, test/kernels/scaled_matmul.py:12-114).  Scales arrive in
// the native layout described in mx_common.h.
//
// Data path per workgroup (one BM x BN tile of C):
//   global --(buffer_load_dwordx4 ... lds, no VGPR staging)--> LDS, two stages
//   LDS --(ds_read_b128, XOR-swizzled 16-byte chunks, conflict free)--> VGPR fragments
//   v_mfma_scale_f32_16x16x128_f8f6f4 with the E8M0 scales of the lane's 32-element K block taken
//   from a VGPR byte selected by op_sel; fp32 accumulators; fused fp32/bf16 epilogue.
//
// MFMA operand roles: the B fragment is passed as the instruction's first matrix and the A fragment
// as the second, so a lane ends up with four CONSECUTIVE columns n of one row m and the epilogue can
// store 8 or 16 contiguous bytes per lane.
//
// Operand layout of v_mfma_scale_f32_16x16x128_f8f6f4 (measured on MI355X with one-hot operands):
//   4-bit formats: lane (r, g) holds row r, K = 32 g + n for nibble n = 0..31 (16 bytes, low nibble
//                  first): exactly the 32-element scale block g.
//   8-bit formats: lane (r, g) holds row r, K = 16 g + b in VGPRs 0-3 (bytes b = 0..15) and
//                  K = 64 + 16 g + b in VGPRs 4-7: two 16-byte pieces, 64 bytes apart in the row.
//   scales:        the scale of block kb (K = 32 kb .. 32 kb + 31) of row r is read from lane
//                  (r, kb), byte op_sel of the scale VGPR, for both formats.  For 8-bit data that is
//                  in general NOT the lane that holds the data.
//   result:        lane (c, g) holds D[4 g + e][c], e = 0..3 (row index = first matrix's row).
#include <stdlib.h>

#include "mx_gemm_tile.h"

namespace mx {
namespace {

// One BM x BN tile of C: `pid` is the workgroup's number among the tiles of the problem, `split` its K slice.
template <class C, typename OutT, bool GROUPED>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, lds_u8* const smem, const int pid, const int split) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, gq = lane >> 4;
  const int wm0 = (wave / C::WGN) * C::WTM, wn0 = (wave % C::WGN) * C::WTN;

  // ---- tile of C owned by this workgroup: XCD-aware, then grouped along M --------------------------
  const int tiles_m = (g.M + C::BM - 1) / C::BM, tiles_n = (g.N + C::BN - 1) / C::BN;
  int tile_m, tile_n, tile_lid;
  {
    const int total = tiles_m * tiles_n;
    // workgroup ids are dealt round-robin to the 8 XCDs (each has its own L2): give every XCD one
    // contiguous range of the logical tile order
    const int xcd = pid & 7, loc = pid >> 3, per = total >> 3, rem = total & 7;
    const int lid = xcd * per + (xcd < rem ? xcd : rem) + loc;
    constexpr int GM = 4;  // row tiles per group (test/kernels/kernel_utils.py:19-29 uses 8; 4 measured equal or faster here)
    const int in_group = GM * tiles_n;
    const int gid = lid / in_group, first_m = gid * GM;
    const int gsz = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    const int in = lid % in_group;
    tile_m = first_m + in % gsz;
    tile_n = in / gsz;
    tile_lid = lid;
  }
  const int m0 = tile_m * C::BM, n0 = tile_n * C::BN;

  // Split-K: blockIdx.y owns the K range [split * g.K, (split + 1) * g.K) of the full problem (g.K is the
  // slice length, a whole number of K-quads), its own slice of the packed scales and its own fp32 partial
  // output; a reduction kernel adds the partials.
  const int ka0 = split * (g.K * C::A_EB / 8), kb0 = split * (g.K * C::B_EB / 8);   // first byte of the slice
  const int Kb_a = ka0 + g.K * C::A_EB / 8, Kb_b = kb0 + g.K * C::B_EB / 8;         // end of the slice in a row
  const int ksteps = (g.K + 127) / 128;
  const int nstages = (ksteps + C::KSUB - 1) / C::KSUB;
  const int KQ = (ksteps + 3) / 4;

  int expert = 0;
  if constexpr (GROUPED) {
    expert = g.sorted_expert_ids[m0 / g.tile_m];
    expert = expert < 0 ? 0 : (expert >= g.num_experts ? g.num_experts - 1 : expert);
  }

  const uint8_t* Bbase = g.B + (GROUPED ? (int64_t)expert * g.b_expert_stride : 0);
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.A, (uint32_t)(g.a_rows * g.lda));
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(Bbase, (uint32_t)((int64_t)g.N * g.ldb));

  // ---- per-thread global offsets of the 16-byte chunks this thread moves each stage -----------------
  // load q of wave w fills LDS slots [(q*NW + w)*64, +64): slot s = (row s / CPR, position s % CPR)
  uint32_t a_voff[C::A_LOADS], b_voff[C::B_LOADS];
  int a_col[C::A_LOADS], b_col[C::B_LOADS];
#pragma unroll
  for (int q = 0; q < C::A_LOADS; ++q) {
    const int slot = (q * C::NW + wave) * 64 + lane;
    const int row = slot / C::A_CPR, pos = slot % C::A_CPR;
    const int col = (pos ^ swz<C::A_CPR>(row)) * 16;
    a_col[q] = col;
    int64_t grow = m0 + row;
    bool ok = grow < g.M;
    if constexpr (GROUPED) {
      const int id = ok ? g.sorted_token_ids[grow] : 0x7FFFFFFF;
      ok = ok && id >= 0 && id < g.num_valid_ids;
      grow = id / g.replicas;
    }
    a_voff[q] = ok ? (uint32_t)(grow * g.lda + col) : kOobOffset;
  }
#pragma unroll
  for (int q = 0; q < C::B_LOADS; ++q) {
    const int slot = (q * C::NW + wave) * 64 + lane;
    const int row = slot / C::B_CPR, pos = slot % C::B_CPR;
    const int col = (pos ^ swz_bperm<C::B_CPR>(row)) * 16;   // the swizzle of the permuted fragment reads below
    b_col[q] = col;
    int64_t grow = n0 + row;
    b_voff[q] = grow < g.N ? (uint32_t)(grow * g.ldb + col) : kOobOffset;
  }

  // One 16-byte-per-lane LDS-DMA load of stage s: idx < A_LOADS moves A rows, the rest B rows.  `live`
  // false (no such stage) turns the load into a zero fill of the idle buffer, which keeps the
  // instruction stream branch-free.
  constexpr int TOTAL_LOADS = C::A_LOADS + C::B_LOADS;
  auto issue_one = [&](int idx, int s, int buf, bool live) {
    lds_u8* const abase = smem + buf * C::STAGE;
    if (idx < C::A_LOADS) {
      const int q = idx, ka = ka0 + s * C::A_RB;
      uint32_t v = a_voff[q];
      if (!live || ka + a_col[q] >= Kb_a) v = kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_void*)(abase + (q * C::NW + wave) * 1024), 16, v,
                                               ka, 0, 0);
    } else {
      const int q = idx - C::A_LOADS, kb = kb0 + s * C::B_RB;
      uint32_t v = b_voff[q];
      if (!live || kb + b_col[q] >= Kb_b) v = kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_void*)(abase + C::A_STAGE + (q * C::NW + wave) * 1024),
                                               16, v, kb, 0, 0);
    }
  };

  // ---- scales: one 16-byte load per lane covers 4 row tiles x 4 K-steps (dword = K-step, byte = tile) ---
  constexpr int AQ = C::MT / 4, BQ = C::NTL / 4;
  // the packed tensors hold ceil(rows / 64) row groups; a tile that hangs over the matrix edge re-reads
  // the last group (its rows are never stored)
  const v4i* const as_ptr = (const v4i*)(g.As + (int64_t)split * g.as_split_stride) + lane;
  const v4i* const bs_ptr = (const v4i*)(g.Bs + (GROUPED ? (int64_t)expert * g.bs_expert_stride : 0) +
                                         (int64_t)split * g.bs_split_stride) + lane;
  const int a_groups = (g.M + 63) / 64, b_groups = (g.N + 63) / 64;
  int a_grp[AQ], b_grp[BQ];
#pragma unroll
  for (int u = 0; u < AQ; ++u) {
    const int grp = (m0 + wm0) / 64 + u;
    a_grp[u] = grp < a_groups ? grp : a_groups - 1;
  }
#pragma unroll
  for (int u = 0; u < BQ; ++u) {
    const int grp = (n0 + wn0) / 64 + u;
    b_grp[u] = grp < b_groups ? grp : b_groups - 1;
  }
  // scales of the current K-quad and, prefetched one quad ahead, of the next
  v4i sa[AQ], sb[BQ], sa_n[AQ], sb_n[BQ];
  auto load_scales = [&](int Q, v4i* da, v4i* db) {
    const int Qc = Q < KQ ? Q : KQ - 1;
#pragma unroll
    for (int u = 0; u < AQ; ++u) da[u] = as_ptr[((int64_t)a_grp[u] * KQ + Qc) * 64];
#pragma unroll
    for (int u = 0; u < BQ; ++u) db[u] = bs_ptr[((int64_t)b_grp[u] * KQ + Qc) * 64];
  };

  v4f acc[C::MT][C::NTL];
#pragma unroll
  for (int i = 0; i < C::MT; ++i)
#pragma unroll
    for (int j = 0; j < C::NTL; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  const int swa = swz<C::A_CPR>(r), swb = swz<C::B_CPR>(r);
  // DMA loads of the next stage are spread over the first half of the MFMA tiles of the current one
  constexpr int LOAD_ITERS = C::MT >= 2 ? C::MT / 2 : 1;
  constexpr int LPI = (TOTAL_LOADS + LOAD_ITERS - 1) / LOAD_ITERS;

  // K is walked in quads of four 128-element steps.  Workgroups that run side by side start at different
  // quads (and wrap around): with power-of-two row pitches all rows of a stage live in the same memory
  // channel, and without the stagger every workgroup would ask that one channel at the same time.
  constexpr int SPQ = 4 / C::KSUB;   // stages per quad
  const int q_start = (g.stagger && ksteps % 4 == 0) ? tile_lid % KQ : 0;
  load_scales(q_start, sa, sb);
#pragma unroll
  for (int idx = 0; idx < TOTAL_LOADS; ++idx) issue_one(idx, q_start * SPQ, 0, true);
  int buf = 0;
  for (int Qi = 0; Qi < KQ; ++Qi) {
    const int Q = Qi + q_start < KQ ? Qi + q_start : Qi + q_start - KQ;
    const int Qn = Q + 1 < KQ ? Q + 1 : 0;
    load_scales(Qn, sa_n, sb_n);
#pragma unroll
    for (int t0 = 0; t0 < 4; t0 += C::KSUB) {
      const int s = Q * SPQ + t0 / C::KSUB;
      const int it = Qi * SPQ + t0 / C::KSUB;        // position in the (rotated) walk
      if (it < nstages) {
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this thread's LDS-DMA of stage s landed
        __syncthreads();                      // everyone's landed; everyone left stage s-1's buffer
        const bool more = it + 1 < nstages;
        const int sn = (t0 / C::KSUB + 1 < SPQ) ? s + 1 : Qn * SPQ;   // stage that follows in the walk
        lds_u8* const atile = smem + buf * C::STAGE + (wm0 + r) * C::A_RB;
        // B rows go to the instruction in the order bperm_row (mx_common.h): tile j of a 64-row group is rows
        // bperm_tile_off(j) + bperm_lane_off(lane % 16), which is also the order of the packed B scales
        lds_u8* const btile = smem + buf * C::STAGE + C::A_STAGE + (wn0 + bperm_lane_off(r)) * C::B_RB;
#pragma unroll
        for (int kk = 0; kk < C::KSUB; ++kk) {
          v8i bf[C::NTL];
#pragma unroll
          for (int j = 0; j < C::NTL; ++j) {
            bf[j] = load_frag<C::B_RB, C::B_EB>(btile, 64 * (j / 4) + bperm_tile_off(j % 4), kk, gq, swb);
          }
#pragma unroll
          for (int i = 0; i < C::MT; ++i) {
            const v8i af = load_frag<C::A_RB, C::A_EB>(atile, 16 * i, kk, gq, swa);
#pragma unroll
            for (int j = 0; j < C::NTL; ++j) {
              acc[i][j] = mfma_scaled<C::BF, C::AF>(bf[j], af, acc[i][j], j % 4, sb[j / 4][t0 + kk], i % 4,
                                                    sa[i / 4][t0 + kk]);
            }
            if (kk == 0 && i < LOAD_ITERS) {
#pragma unroll
              for (int l = 0; l < LPI; ++l)
                if (i * LPI + l < TOTAL_LOADS) issue_one(i * LPI + l, sn, buf ^ 1, more);
            }
            // keep the DMA loads in the tile iteration they were written in; everything else may move
            __builtin_amdgcn_sched_barrier(0x78F);
          }
        }
        buf ^= 1;
      }
    }
#pragma unroll
    for (int u = 0; u < AQ; ++u) sa[u] = sa_n[u];
#pragma unroll
    for (int u = 0; u < BQ; ++u) sb[u] = sb_n[u];
  }

  // ---- epilogue: lane (r, gq) of tile (i, j) holds row m0 + wm0 + 16 i + r, columns
  // n0 + wn0 + 64 (j / 4) + bperm_tile_off(j % 4) + 8 gq .. + 3 -----------------------------------------------
  OutT* const Cp = (OutT*)g.C + (int64_t)split * g.c_split_stride;
  const bool vec_ok = (g.ldc % 4 == 0) && (((uintptr_t)g.C) % 16 == 0) && (g.c_split_stride % 4 == 0);
  const bool accumulate = g.accumulate != 0;
#pragma unroll
  for (int i = 0; i < C::MT; ++i) {
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
    for (int j = 0; j < C::NTL; ++j) {
      const int n = n0 + wn0 + 64 * (j / 4) + bperm_tile_off(j % 4) + 8 * gq;
      if (n >= g.N) continue;
      v4f v = acc[i][j];
      if constexpr (GROUPED) v *= w;
      store4<OutT>(Cp + orow * g.ldc + n, v, accumulate, g.N - n, vec_ok);
    }
  }
}

template <class C, typename OutT, bool GROUPED>
__global__ __launch_bounds__(C::NT) void gemm_kernel(const GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_generic[];
  gemm_tile<C, OutT, GROUPED>(g, (lds_u8*)smem_generic, blockIdx.x, blockIdx.y);
}

// ---- list of problems: persistent workgroups walk the concatenated tile list -----------------------------------
constexpr int kListMax = 32;
struct ListProblem {
  const uint8_t* A; const uint8_t* B; const uint32_t* As; const uint32_t* Bs; void* C;
  int64_t lda, ldb, ldc;
  int32_t M, N, K, accumulate;
};
struct GemmList {
  ListProblem p[kListMax];
  int32_t first_tile[kListMax + 1];
  int32_t n, a_fmt, b_fmt, c_dtype;
};

template <class C, typename OutT>
__global__ __launch_bounds__(C::NT) void gemm_list_kernel(const GemmList gl) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_generic[];
  const int total = gl.first_tile[gl.n];
  for (int t = blockIdx.x; t < total; t += gridDim.x) {   // uniform per workgroup
    int i = 0;
    while (i + 1 < gl.n && t >= gl.first_tile[i + 1]) ++i;
    const ListProblem& q = gl.p[i];
    GemmArgs g = {};
    g.A = q.A; g.B = q.B; g.As = q.As; g.Bs = q.Bs; g.C = q.C;
    g.lda = q.lda; g.ldb = q.ldb; g.ldc = q.ldc;
    g.M = q.M; g.N = q.N; g.K = q.K;
    g.a_fmt = gl.a_fmt; g.b_fmt = gl.b_fmt; g.c_dtype = gl.c_dtype; g.accumulate = q.accumulate;
    g.a_rows = q.M; g.replicas = 1;
    gemm_tile<C, OutT, false>(g, (lds_u8*)smem_generic, t - gl.first_tile[i], 0);
    // the tile's trailing (zero-fill) DMA has left the queue and every wave is done with the LDS stages before
    // the next tile's loads reuse them
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  }
}

template <class C, typename OutT>
int launch_list_one(const GemmList& gl, hipStream_t stream) {
  auto kern = gemm_list_kernel<C, OutT>;
  static int attr_done = 0;   // benign race: the attribute call is idempotent
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess)
      return set_error(MX_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", C::LDS_BYTES, hipGetErrorString(e));
    attr_done = 1;
  }
  const int total = gl.first_tile[gl.n];
  if (total <= 0) return MX_OK;
  const int grid = total < 1024 ? total : 1024;   // 128 x 128 tiles: up to four workgroups per CU are resident
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(C::NT), C::LDS_BYTES, stream, gl);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "gemm_list_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

template <class C, typename OutT, bool GROUPED>
int launch_one(const GemmArgs& g, hipStream_t stream) {
  auto kern = gemm_kernel<C, OutT, GROUPED>;
  static int attr_done = 0;   // benign race: the attribute call is idempotent
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       C::LDS_BYTES);
    if (e != hipSuccess)
      return set_error(MX_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", C::LDS_BYTES,
                       hipGetErrorString(e));
    attr_done = 1;
  }
  const int64_t tiles = (int64_t)((g.M + C::BM - 1) / C::BM) * ((g.N + C::BN - 1) / C::BN);
  if (tiles <= 0) return MX_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)(g.k_splits > 1 ? g.k_splits : 1)), dim3(C::NT),
                     C::LDS_BYTES, stream, g);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "gemm_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

template <int BM, int BN, int WGM, int WGN>
int launch_fmt(const GemmArgs& g, hipStream_t stream) {
  const bool grouped = g.sorted_token_ids != nullptr;
  GemmArgs gs = g;
#define MX_CASE(AFMT, BFMT)                                                                        \
  if (g.a_fmt == AFMT && g.b_fmt == BFMT) {                                                        \
    using C = Cfg<AFMT, BFMT, BM, BN, WGM, WGN>;                                                   \
    if (g.c_dtype == MX_F32)                                                                       \
      return grouped ? launch_one<C, float, true>(gs, stream) : launch_one<C, float, false>(gs, stream); \
    return grouped ? launch_one<C, uint16_t, true>(gs, stream)                                      \
                   : launch_one<C, uint16_t, false>(gs, stream);                                    \
  }
  MX_CASE(MX_E4M3, MX_E4M3)
  MX_CASE(MX_E5M2, MX_E5M2)
  MX_CASE(MX_E2M1, MX_E2M1)
  MX_CASE(MX_E4M3, MX_E2M1)
#undef MX_CASE
  return set_error(MX_ERR_DTYPE, "MFMA kernel: unsupported element format pair (%d, %d)", g.a_fmt,
                   g.b_fmt);
}

}  // namespace

int launch_gemm_mfma_list(const GemmArgs* problems, int n, hipStream_t stream) {
  for (int i0 = 0; i0 < n; i0 += kListMax) {
    GemmList gl = {};
    int64_t total = 0;
    for (int i = i0; i < n && i < i0 + kListMax; ++i) {
      const GemmArgs& g = problems[i];
      if (g.a_fmt != problems[0].a_fmt || g.b_fmt != problems[0].b_fmt || g.c_dtype != problems[0].c_dtype ||
          g.sorted_token_ids || g.k_splits > 1)
        return set_error(MX_ERR_INVALID, "gemm list: problems of one launch must share formats and be plain products");
      ListProblem& q = gl.p[gl.n];
      q.A = g.A; q.B = g.B; q.As = g.As; q.Bs = g.Bs; q.C = g.C;
      q.lda = g.lda; q.ldb = g.ldb; q.ldc = g.ldc;
      q.M = g.M; q.N = g.N; q.K = g.K; q.accumulate = g.accumulate;
      gl.first_tile[gl.n] = (int32_t)total;
      total += (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
      if (total > 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "gemm list: too many tiles");
      ++gl.n;
    }
    gl.first_tile[gl.n] = (int32_t)total;
    gl.a_fmt = problems[0].a_fmt; gl.b_fmt = problems[0].b_fmt; gl.c_dtype = problems[0].c_dtype;
    int rc = MX_ERR_DTYPE;
#define MX_CASE(AFMT, BFMT)                                                                       \
    if (gl.a_fmt == AFMT && gl.b_fmt == BFMT) {                                                     \
      using C = Cfg<AFMT, BFMT, 128, 128, 2, 2>;                                                    \
      rc = gl.c_dtype == MX_F32 ? launch_list_one<C, float>(gl, stream) : launch_list_one<C, uint16_t>(gl, stream); \
    }
    MX_CASE(MX_E4M3, MX_E4M3)
    MX_CASE(MX_E5M2, MX_E5M2)
    MX_CASE(MX_E2M1, MX_E2M1)
    MX_CASE(MX_E4M3, MX_E2M1)
#undef MX_CASE
    if (rc == MX_ERR_DTYPE) return set_error(MX_ERR_DTYPE, "gemm list: unsupported element format pair (%d, %d)", gl.a_fmt, gl.b_fmt);
    if (rc != MX_OK) return rc;
  }
  return MX_OK;
}

int launch_gemm_mfma(const GemmArgs& g, int kernel_id, hipStream_t stream) {
  if (g.c_dtype != MX_F32 && g.c_dtype != MX_BF16)
    return set_error(MX_ERR_DTYPE, "MFMA kernel: output dtype %d not supported", g.c_dtype);
  switch (kernel_id) {
    case MX_KERNEL_MFMA_128x128: return launch_fmt<128, 128, 2, 2>(g, stream);
    case MX_KERNEL_MFMA_256x256: return launch_fmt<256, 256, 2, 4>(g, stream);
    case MX_KERNEL_MFMA_256x256_W4: return launch_fmt<256, 256, 2, 2>(g, stream);
    case MX_KERNEL_MFMA_PINGPONG: return launch_gemm_pingpong(g, stream);
    case MX_KERNEL_MFMA_PINGPONG32: return launch_gemm_pingpong32(g, stream);
    case MX_KERNEL_MFMA_W4_PERSISTENT: return launch_gemm_w4(g, stream);
  }
  return set_error(MX_ERR_INVALID, "unknown MFMA kernel id %d", kernel_id);
}

}  // namespace mx
