// Skinny-M ("decode") block-scaled GEMM: C[M<=32, N] = X[M, K] (8-bit MX) x W[N, K] (MXFP4) ^T.
//
// The problem is bound by streaming W (and its scales) from HBM exactly once, so the kernel is organised around
// long contiguous reads and many bytes in flight, not around tile reuse:
//   * a workgroup of 8 waves takes every gridDim.x-th 16-row tile of W (64 KiB at K = 8192); the waves are
//     4 K-slices x 2 halves of M (16 rows of X each): wave (q, mh) multiplies K-slice q of every tile by rows
//     16 mh .. of X, and loads rows 8 mh .. 8 mh + 7 of the slice;
//   * W and its E8M0 scales go global -> LDS with buffer_load ... lds (no VGPR staging), one DMA instruction per
//     KiB of one weight row (two rows at K <= 4096); two tiles per workgroup are in flight (136 KiB per CU) while
//     the previous one is multiplied; one barrier tells that a tile has landed, one that its slot may be refilled;
//   * each wave keeps its K-slice of X (and of the X scales) resident in VGPRs for the whole kernel, in the 8-bit
//     MFMA operand layout (bytes 16 g .. 16 g + 15 and 64 + 16 g .. of each K-step for lane group g); X reaches the
//     registers through LDS, see the kernel;
//   * v_mfma_scale_f32_16x16x128_f8f6f4 with mixed formats (W as FP4 first matrix, X as FP8 second matrix); W
//     fragments are read from LDS (16-byte chunks XOR-swizzled by row: conflict free), the scale bytes of the
//     lane's blocks are packed one register per four K-steps for op_sel to walk;
//   * the 4 partial sums of a tile meet in LDS and two waves convert and store them while the next tiles stream.
// K may be any multiple of 512 up to 8192: the kernel is instantiated for K-slices of 1024 (K <= 4096) and 2048
// elements, and lanes whose bytes lie beyond K fetch nothing (their LDS bytes arrive as zeros, which multiply to
// nothing), so a shorter K costs LDS reads and MFMAs of the padding but no memory traffic.  (A variant whose 8
// waves all split K and need no barrier while streaming measured 5 - 25 % slower at every K and is gone.)
#include <stdlib.h>

#include "mx_common.h"

namespace mx {
namespace {

typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(3))) const v4i lds_cv4i;
typedef __attribute__((address_space(3))) v4f lds_v4f;

constexpr int kWaves = 8;
constexpr uint32_t kOob = 0x80000000u;         // beyond num_records of the descriptors built here

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// ---- configuration for K-slices of SPW K-steps (K <= 4 * SPW * 128) ------------------------------------------------
// The two waves of a K-slice multiply the same
// weight fragments by their own half of X, so a tile is shared through LDS: each of the two loads half of
// the slice's rows, one workgroup barrier tells that a tile has landed and one that its slot may be
// refilled.  LDS slot of a tile: [K-slice][row][slice bytes] (16-byte chunks XOR-swizzled by row), then
// [row][K/32] scale bytes; two slots, i.e. two tiles in flight per workgroup.
template <int SPW>
struct DecodeCfg {
  static constexpr int SLB = SPW * 64;            // bytes of a weight row inside one K-slice
  static constexpr int LPR = SLB / 16;            // lanes (16-byte chunks) per row of a slice
  static constexpr int RPI = 64 / LPR;            // rows per DMA instruction
  static constexpr int WIW = 16 / RPI / 2;        // weight DMA instructions per wave and tile
  static constexpr int SROW = SPW * 16;           // scale bytes per weight row (K / 32)
  static constexpr int LS = SROW / 16;            // lanes per scale row
  // XOR term of a scale row's 16-byte pieces in LDS: rows that start in the same bank differ in it
  __device__ static constexpr int sswz(int row) { return (row * SROW / 256) % LS; }
  static constexpr int S_INSTR = 16 * SROW / 1024;   // scale DMA instructions per tile (waves 0 .. S_INSTR-1)
  static constexpr int W_BYTES = 4 * 16 * SLB;
  static constexpr int SLOT = W_BYTES + 16 * SROW;
  static constexpr int RING = 2 * SLOT;
  static constexpr int RED = kWaves * 64 * 16;       // partial sums of one tile: [wave][lane] float4
  // Staging of X before the stream starts: XNB round buffers of 4 KiB per wave (16 rows x 256 bytes).  Tile 0 is in
  // flight to slot 1 meanwhile, so the buffers sit inside slot 0 if that is large enough, else behind the reduction
  // buffers; the X scales (1 KiB per wave) use the reduction buffers, which are idle until tile 0 is done.
  static constexpr int XNB = 2;
  static constexpr int XSTAGE = kWaves * XNB * 4096;
  static constexpr int XSTAGE_OFF = XSTAGE <= SLOT ? 0 : RING + 2 * RED;
  static constexpr int XSCALE_OFF = RING;
  static constexpr int LDS_BYTES = XSTAGE <= SLOT ? RING + 2 * RED : RING + 2 * RED + XSTAGE;
  static_assert(kWaves * 1024 <= 2 * RED, "X scale staging");
};

// The weight and scale DMA of one wave for one tile.  Instruction j of the wave covers rows
// rbase + j * RPI ... of the tile; lane offsets: row_off = (lane / LPR) * ldw, chunk_off = the lane's 16-byte
// chunk position already XORed with its row inside the instruction (plus the K-slice's byte offset); the
// instruction's first row enters the swizzle as one more XOR (rbase + RPI * j and lane / LPR share no bits).
template <int SPW>
__device__ inline void issue_tile_dma2(const uint8_t* W, uint32_t wbytes, const uint8_t* S, uint32_t sbytes,
                                       lds_u8* wdst, lds_u8* sdst, uint32_t row_off, uint32_t chunk_off, int rbase,
                                       uint32_t soff, int wsoff, int ldw, int ssoff, bool with_scales,
                                       uint32_t row_bytes) {
  using Cf = DecodeCfg<SPW>;
  const __amdgpu_buffer_rsrc_t rsW = make_rsrc(W, wbytes), rsS = make_rsrc(S, sbytes);
#pragma unroll
  for (int j = 0; j < Cf::WIW; ++j) {
    const int r0 = rbase + j * Cf::RPI;
    const uint32_t off = chunk_off ^ (uint32_t)((r0 & 15) << 4);     // byte of the row this lane fetches
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsW, (lds_void*)(wdst + j * 1024), 16,
                                             off < row_bytes ? row_off + off : kOob, wsoff + r0 * ldw, 0, 0);
  }
  if (with_scales)   // uniform per wave
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsS, (lds_void*)sdst, 16, soff, ssoff, 0, 0);
}

// The 4 LDS-DMA loads of one staging round of a wave: 256 bytes of each of 16 consecutive rows of X (4 rows per
// instruction), row rr to dst + rr * 256
// (voff[j]: lane offset of instruction j; cb[j]: the byte inside the round's 256 that the lane fetches; bytes at or
// beyond kleft, the end of the row, are not fetched and arrive as zeros)
__device__ inline void issue_x_round(const uint8_t* X, uint32_t xbytes, lds_u8* dst, const uint32_t* voff, const int* cb,
                                     int kleft, int soff0, int ldx) {
  const __amdgpu_buffer_rsrc_t rsX = make_rsrc(X, xbytes);
#pragma unroll
  for (int j = 0; j < 4; ++j)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsX, (lds_void*)(dst + j * 1024), 16, cb[j] < kleft ? voff[j] : kOob,
                                             soff0 + 4 * j * ldx, 0, 0);
}
__device__ inline void issue_xs_dma(const uint8_t* Xs, uint32_t bytes, lds_u8* dst, uint32_t voff, int soff) {
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(Xs, bytes);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)dst, 16, voff, soff, 0, 0);
}

template <int XF, int SPW, typename OutT>
__global__ __launch_bounds__(kWaves * 64) void decode_kernel(const DecodeArgs d) {
  using Cf = DecodeCfg<SPW>;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_generic[];
  lds_u8* const smem = (lds_u8*)smem_generic;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = wave & 3, mh = wave >> 2;      // K-slice, half of M
  const int r = lane & 15, gq = lane >> 4;
  const bool with_scales = wave < Cf::S_INSTR;

  // ---- per-lane DMA offsets inside a tile --------------------------------------------------------------
  // (descriptor ranges end with the last row's last byte of this K range: the operands may be K-chunks of wider rows)
  const uint32_t wbytes = (uint32_t)((int64_t)(d.N - 1) * d.ldw + d.K / 2);
  const uint32_t sbytes = (uint32_t)((int64_t)(d.N - 1) * d.ldws + d.K / 32);
  const int rl = lane / Cf::LPR;                 // row of the lane inside one DMA instruction
  const uint32_t row_off = (uint32_t)(rl * d.ldw);
  const uint32_t chunk_off = (uint32_t)((((lane % Cf::LPR) ^ rl) << 4) + q * Cf::SLB);   // SLB: no bits below 512
  // a scale row is SROW = 256 (128) bytes in LDS, so every (second) row starts in the same bank: the 16-byte
  // pieces of a row are XOR-swizzled by the row like the weight chunks, and the 16 rows a fragment read touches
  // sit in 16 different bank groups
  const int srow = wave * (64 / Cf::LS) + lane / Cf::LS;
  const int spiece = ((lane % Cf::LS) ^ Cf::sswz(srow)) * 16;    // byte of the scale row this lane fetches
  const uint32_t soff = spiece < d.K / 32 ? (uint32_t)(srow * d.ldws + spiece) : kOob;
  // Tiles of this workgroup: local tile i is tile t_first + i G (16 consecutive weight rows), so that the workgroups
  // together read one contiguous window of G tiles at a time.  Workgroup ids go round-robin over the 8 XCDs; XCD x
  // takes the x-th eighth of every window, so that every XCD reads from all address slices instead of always the
  // same eighth of them (measured 1.1 us of 29 at the 28672 x 8192 weights; two windows of 8-row half tiles, which
  // a pure streaming test prefers, measure 2 us slower here).
  const int tiles = d.N / 16;
  const int G = gridDim.x;
  const int t_first = G % 8 == 0 ? (blockIdx.x % 8) * (G / 8) + blockIdx.x / 8 : blockIdx.x;
  const int t_count = t_first < tiles ? (tiles - t_first + G - 1) / G : 0;
  auto issue = [&](int i, int slot) {          // this wave's share of local tile i
    const int tile = t_first + i * G;
    lds_u8* const base = smem + slot * Cf::SLOT;
    issue_tile_dma2<SPW>(d.W, wbytes, d.Ws, sbytes, base + q * (16 * Cf::SLB) + mh * Cf::WIW * 1024,
                         base + Cf::W_BYTES + wave * 1024, row_off, chunk_off, mh * Cf::WIW * Cf::RPI, soff,
                         tile * 16 * (int)d.ldw, (int)d.ldw, tile * 16 * (int)d.ldws, with_scales, (uint32_t)(d.K / 2));
  };

  if (t_count == 0) return;                    // uniform per workgroup

  // ---- resident X: rows 16 mh + r, K-steps q SPW .. of it ------------------------------------------------------
  // X comes through LDS: a DMA instruction reads 256 contiguous bytes of each of 4 rows of X, and the wave then picks
  // its operand registers out of its own staging area.  (Loading the operand layout straight from memory, 16 rows
  // x 64 bytes per instruction and every workgroup the same 264 KiB, keeps the texture-address unit and L2 busy for
  // 6 us at the 32 x 8192 activations; this way the 256 KiB cross the CU's 64-byte/clock memory port in 3 us.)  A round
  // is two K-steps: 16 rows x 256 bytes per wave, 16-byte chunks XOR-swizzled by row; two rounds are in flight.  Lanes
  // whose row is at or beyond M fetch nothing (offset beyond the descriptor) and their bytes arrive as zeros (scale
  // byte 0 = 2^-127).
  // The DMA of tile 0 is requested first: the memory pipe returns data in request order for the whole CU, so X
  // arrives behind it, but HBM has something to do meanwhile (0.7 us faster than staging X first); with both first
  // tiles in flight there would be no room in LDS to stage X.
  v8i xf[SPW];
  int xs[SPW / 4];
  {
    constexpr int XR = SPW / 2;                       // rounds
    issue(0, 1);                                       // tile i lives in slot (i + 1) % 2
    lds_u8* const xst = smem + Cf::XSTAGE_OFF + wave * (Cf::XNB * 4096);
    lds_u8* const xsst = smem + Cf::XSCALE_OFF + wave * 1024;
    const uint32_t xbytes = (uint32_t)((int64_t)(d.M - 1) * d.ldx + d.K);
    uint32_t xvo[4];                                  // lane offsets of the 4 DMA instructions of a round
    int xcb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      xcb[j] = ((lane & 15) ^ (4 * j + (lane >> 4))) << 4;
      // the row term 16 mh + 4 j of the address travels in the instruction's scalar offset, which the descriptor's
      // range check does not see: a lane whose row is at or beyond M is masked here instead
      xvo[j] = 16 * mh + 4 * j + (lane >> 4) < d.M ? (uint32_t)((lane >> 4) * d.ldx + xcb[j]) : kOob;
    }
    const int xso = 16 * mh * (int)d.ldx + q * SPW * 128;
    const int xk = d.K - q * SPW * 128;               // bytes of a row of X from the start of this wave's K-slice on
    // the wave's own X scales: 16 rows x SPW * 4 bytes, one instruction
    {
      constexpr int LPRS = SPW * 4 / 16;              // lanes per row
      const int srw = lane / LPRS;
      const bool sok = srw < 16 && 16 * mh + srw < d.M && q * SPW * 4 + (lane % LPRS) * 16 < d.K / 32;
      issue_xs_dma(d.Xs, (uint32_t)((int64_t)(d.M - 1) * d.ldxs + d.K / 32), xsst,
                   sok ? (uint32_t)(srw * d.ldxs + (lane % LPRS) * 16) : kOob, 16 * mh * (int)d.ldxs + q * SPW * 4);
    }
#pragma unroll
    for (int h = 0; h < Cf::XNB && h < XR; ++h)
      issue_x_round(d.X, xbytes, xst + h * 4096, xvo, xcb, xk - h * 256, xso + h * 256, (int)d.ldx);
#pragma unroll
    for (int h = 0; h < XR; ++h) {
      static_assert(Cf::XNB == 2, "wait counts below");
      if (h + 1 < XR) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);   // round h + 1 may stay in flight
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      asm volatile("" ::: "memory");
      lds_u8* const row = xst + (h % Cf::XNB) * 4096 + r * 256;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const v4i lo = *(lds_cv4i*)(row + (((s2 * 8 + gq) ^ r) << 4));
        const v4i hi = *(lds_cv4i*)(row + (((s2 * 8 + 4 + gq) ^ r) << 4));
        xf[h * 2 + s2] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
      if (h == 0) {                                    // the scales landed before round 0
#pragma unroll
        for (int u = 0; u < SPW / 4; ++u) {
          const v4i raw = *(lds_cv4i*)(xsst + r * (SPW * 4) + u * 16);
          uint32_t pk = 0;
#pragma unroll
          for (int t = 0; t < 4; ++t) pk |= (((uint32_t)raw[t] >> (8 * gq)) & 0xFFu) << (8 * t);
          xs[u] = (int)pk;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // round h + XNB (or the weight stream) overwrites the buffer
      if (h + Cf::XNB < XR)
        issue_x_round(d.X, xbytes, xst + (h % Cf::XNB) * 4096, xvo, xcb, xk - (h + Cf::XNB) * 256,
                      xso + (h + Cf::XNB) * 256, (int)d.ldx);
    }
    __syncthreads();                                   // the weight slots overlap the other waves' staging areas
    if (t_count > 1) issue(1, 0);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- per tile: partial sums of the 4 K-slices meet in LDS and leave while the next tiles stream in -------
  const bool vec_ok = (d.ldc % 4 == 0) && (((uintptr_t)d.C) % 16 == 0);
  auto reduce_store = [&](int k) {   // local tile k; threads 0 .. 127: half of M = tid / 64, lane l = tid % 64
    lds_v4f* const red = (lds_v4f*)(smem + Cf::RING + (k & 1) * Cf::RED);
    const int h = tid >> 6, l = tid & 63;
    v4f sum = red[(h * 4 + 0) * 64 + l];
#pragma unroll
    for (int w = 1; w < 4; ++w) sum += red[(h * 4 + w) * 64 + l];
    // lane (c, g) holds C[16 h + c][16 tile + 4 g + e], e = 0..3
    const int row = 16 * h + (l & 15);
    if (row >= d.M) return;
    OutT* c = (OutT*)d.C + (int64_t)row * d.ldc + (t_first + k * G) * 16 + 4 * (l >> 4);
    if constexpr (sizeof(OutT) == 4) {
      if (vec_ok) {
        if (d.accumulate) sum += *(const v4f*)c;
        *(v4f*)c = sum;
      } else {
        for (int e = 0; e < 4; ++e) c[e] = d.accumulate ? c[e] + sum[e] : sum[e];
      }
    } else {
      if (vec_ok) {
        if (d.accumulate) {
          const uint2 old = *(const uint2*)c;
          sum.x += bf16_to_f32((uint16_t)old.x); sum.y += bf16_to_f32((uint16_t)(old.x >> 16));
          sum.z += bf16_to_f32((uint16_t)old.y); sum.w += bf16_to_f32((uint16_t)(old.y >> 16));
        }
        uint2 o;
        o.x = (uint32_t)f32_to_bf16(sum.x) | ((uint32_t)f32_to_bf16(sum.y) << 16);
        o.y = (uint32_t)f32_to_bf16(sum.z) | ((uint32_t)f32_to_bf16(sum.w) << 16);
        *(uint2*)c = o;
      } else {
        for (int e = 0; e < 4; ++e)
          c[e] = f32_to_bf16(d.accumulate ? bf16_to_f32(c[e]) + sum[e] : sum[e]);
      }
    }
  };

  for (int i = 0; i < t_count; ++i) {   // uniform per workgroup
    // this wave's share of tile i has landed (its share of tile i + 1 may stay in flight; the output store
    // that waves 0 and 1 issued after it is younger still, so they wait for the first load of tile i + 1 as
    // well -- measured: allowing for that store changes nothing, and counting it exactly would depend on
    // which form of the epilogue ran) ...
    if (i + 1 < t_count) {
      if (with_scales) __builtin_amdgcn_s_waitcnt(0x0F70 | (Cf::WIW + 1));
      else __builtin_amdgcn_s_waitcnt(0x0F70 | Cf::WIW);
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __builtin_amdgcn_sched_barrier(0);
    // ... and so has everybody else's; the partial sums of tile i - 1 are all in LDS as well
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // all of the tile's fragments and scales into registers, so that the slot can be refilled before the
    // multiplications start.  The scales first, packed to the lane's own byte of each K-step (one register
    // per four K-steps): with the 16 raw scale registers alive next to the fragments the kernel would spill,
    // and a spill reload queues behind the DMA just issued.
    lds_u8* const wt = smem + ((i + 1) & 1) * Cf::SLOT + q * (16 * Cf::SLB) + r * Cf::SLB;
    lds_u8* const st = smem + ((i + 1) & 1) * Cf::SLOT + Cf::W_BYTES + r * Cf::SROW;
    int ws[SPW / 4];
    v4i w[SPW];
    {
#pragma unroll
      for (int h = 0; h < SPW / 4; ++h) {
        const v4i sc = *(lds_cv4i*)(st + (((q * (SPW / 4) + h) ^ Cf::sswz(r)) << 4));
        uint32_t pk = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) pk |= (((uint32_t)sc[t] >> (8 * gq)) & 0xFFu) << (8 * t);
        ws[h] = (int)pk;
      }
      __builtin_amdgcn_sched_barrier(0);
      // chunk (4 s + g) ^ r = 16 (s / 4) + (4 ((s % 4) ^ (r / 4)) + (g ^ (r % 4))): four lane-dependent
      // addresses, the rest is an immediate offset
      lds_u8* wk[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) wk[k] = wt + ((4 * (k ^ (r >> 2)) + (gq ^ (r & 3))) << 4);
#pragma unroll
      for (int s = 0; s < SPW; ++s) w[s] = *(lds_cv4i*)(wk[s & 3] + (s >> 2) * 256);
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    if (i + 2 < t_count) issue(i + 2, (i + 1) & 1);
    __builtin_amdgcn_sched_barrier(0);
    if (i > 0 && wave < 2) reduce_store(i - 1);   // uniform per wave
    v4f acc[2] = {(v4f){0.f, 0.f, 0.f, 0.f}, (v4f){0.f, 0.f, 0.f, 0.f}};   // even / odd K-steps: two MFMA chains
    {
#pragma unroll
      for (int s = 0; s < SPW; ++s) {
        const v8i wf = {w[s].x, w[s].y, w[s].z, w[s].w, 0, 0, 0, 0};
        v4f& a = acc[s & 1];
        if (s % 4 == 0)
          a = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[s], a, MX_E2M1, XF, 0, ws[s / 4], 0, xs[s / 4]);
        else if (s % 4 == 1)
          a = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[s], a, MX_E2M1, XF, 1, ws[s / 4], 1, xs[s / 4]);
        else if (s % 4 == 2)
          a = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[s], a, MX_E2M1, XF, 2, ws[s / 4], 2, xs[s / 4]);
        else
          a = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[s], a, MX_E2M1, XF, 3, ws[s / 4], 3, xs[s / 4]);
      }
    }
    ((lds_v4f*)(smem + Cf::RING + (i & 1) * Cf::RED))[wave * 64 + lane] = acc[0] + acc[1];
  }
  __syncthreads();
  if (wave < 2) reduce_store(t_count - 1);
}

template <int XF, int SPW, typename OutT>
int launch_decode_k(const DecodeArgs& d, int grid, hipStream_t stream) {
  using Cf = DecodeCfg<SPW>;
  auto kern = decode_kernel<XF, SPW, OutT>;
  static int attr_done = 0;   // benign race: the attribute call is idempotent
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, Cf::LDS_BYTES);
    if (e != hipSuccess)
      return set_error(MX_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", Cf::LDS_BYTES, hipGetErrorString(e));
    attr_done = 1;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kWaves * 64), Cf::LDS_BYTES, stream, d);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(MX_ERR_LAUNCH, "decode_kernel launch: %s", hipGetErrorString(e));
  return MX_OK;
}

template <int XF>
int launch_decode_x(const DecodeArgs& d, int grid, hipStream_t stream) {
  if (d.K > 4096)
    return d.c_dtype == MX_F32 ? launch_decode_k<XF, 16, float>(d, grid, stream)
                               : launch_decode_k<XF, 16, uint16_t>(d, grid, stream);
  return d.c_dtype == MX_F32 ? launch_decode_k<XF, 8, float>(d, grid, stream)
                             : launch_decode_k<XF, 8, uint16_t>(d, grid, stream);
}

}  // namespace


int launch_gemm_decode(const DecodeArgs& d, hipStream_t stream) {
  if (d.w_fmt != MX_E2M1) return set_error(MX_ERR_DTYPE, "decode kernel: weights must be MX_E2M1");
  if (d.x_fmt != MX_E4M3 && d.x_fmt != MX_E5M2) return set_error(MX_ERR_DTYPE, "decode kernel: activations must be 8-bit");
  if (d.M < 1 || d.M > 32) return set_error(MX_ERR_SHAPE, "decode kernel: M must be in 1..32");
  if (d.K % 512 != 0 || d.K > kWaves * 8 * 128)
    return set_error(MX_ERR_SHAPE, "decode kernel: K must be a multiple of 512 and at most %d", kWaves * 8 * 128);
  if (d.N % 16 != 0) return set_error(MX_ERR_SHAPE, "decode kernel: N must be a multiple of 16");
  if (((uintptr_t)d.X | (uintptr_t)d.Xs | (uintptr_t)d.W | (uintptr_t)d.Ws | (uintptr_t)d.ldx | (uintptr_t)d.ldxs |
       (uintptr_t)d.ldw | (uintptr_t)d.ldws) % 16 != 0)
    return set_error(MX_ERR_LAYOUT, "decode kernel: operands, scales and their row pitches must be 16-byte aligned");
  if ((int64_t)d.N * d.ldw >= ((int64_t)1 << 31) || (int64_t)d.N * d.ldws >= ((int64_t)1 << 31))
    return set_error(MX_ERR_LAYOUT, "decode kernel: W spans 2 GiB or more");
  if (d.c_dtype != MX_F32 && d.c_dtype != MX_BF16) return set_error(MX_ERR_DTYPE, "decode kernel: bad output dtype");
  const int tiles = d.N / 16;
  const int grid = tiles < 256 ? tiles : 256;
  if (grid == 0) return MX_OK;
  return d.x_fmt == MX_E4M3 ? launch_decode_x<MX_E4M3>(d, grid, stream) : launch_decode_x<MX_E5M2>(d, grid, stream);
}

}  // namespace mx
