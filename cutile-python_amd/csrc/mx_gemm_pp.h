// Pieces shared by the persistent ping-pong GEMM kernels (mx_gemm_pp.hip: 16x16x128 MFMA tiles, all element
// formats; mx_gemm_pp32.hip: 32x32x64 MFMA tiles, 8-bit formats): LDS budget, tile walk, launch helpers.
#pragma once
#include "mx_gemm_tile.h"

namespace mx {

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
constexpr int vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

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
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

// Tiles a workgroup walks: linear tile ids first, first + step, ... below end.  Linear ids map to
// (tile row, tile column) in groups of 4 tile rows walked column by column (the 32 tiles an XCD works on at a
// time are 4 tile rows x 8 tile columns, which its L2 serves).
struct TileWalk {
  int first, step, end, tiles_m, tiles_n;
  __device__ void origin(int lid, int& m0, int& n0) const {
    constexpr int GM = 4;   // measured: 4 rows is 1 - 3 % faster than 8 (2, 3, 6, 16 are slower than either)
    const int in_group = GM * tiles_n;
    const int gid = lid / in_group, first_m = gid * GM;
    const int gsz = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    const int in = lid % in_group;
    m0 = (first_m + in % gsz) * 256;
    n0 = (in / gsz) * 256;
  }
};

// Workgroup ids are dealt round-robin to the 8 XCDs (each with its own L2): XCD x owns a contiguous range of
// linear tile ids, and its workgroups walk that range with a stride of their count.
__device__ inline TileWalk make_tile_walk(int M, int N) {
  TileWalk walk;
  walk.tiles_m = (M + 255) / 256;
  walk.tiles_n = (N + 255) / 256;
  const int total = walk.tiles_m * walk.tiles_n;
  const int pid = blockIdx.x, grid = gridDim.x;
  const int xcd = pid & 7, loc = pid >> 3, per = total >> 3, rem = total & 7;
  const int start = xcd * per + (xcd < rem ? xcd : rem);
  const int count = per + (xcd < rem ? 1 : 0);
  walk.step = (grid - xcd + 7) >> 3;   // workgroups of this XCD
  walk.first = start + loc;
  walk.end = start + count;
  return walk;
}

inline int num_cus() {
  static int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
    return n;
  }();
  return cus;
}

// grid of a persistent ping-pong launch: one workgroup per CU walking several tiles when the stage pipeline can
// run across tile boundaries (at least two stages per tile, whole K-quads); otherwise one workgroup per tile
inline int64_t pp_grid(int M, int N, int K, int ksub) {
  const int64_t tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  const int ksteps = (K + 127) / 128;
  const int nstages = (ksteps + ksub - 1) / ksub;
  const bool can_walk = nstages >= 2 && ksteps % 4 == 0;
  return (can_walk && tiles > num_cus()) ? num_cus() : tiles;
}

}  // namespace mx
