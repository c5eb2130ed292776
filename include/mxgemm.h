/*
 * mxgemm.h -- C ABI of libmxgemm.so: block-scaled (MX) matrix multiply for AMD MI355X (gfx950).
 *
 * Plain C, plain pointers and sizes; no C++ or framework types cross this boundary.  Every entry
 * point enqueues work on the given hipStream_t (passed as void*; NULL = the null stream) and
 * returns without synchronising.  Return value: 0 on success, a negative MX_ERR_* otherwise; the
 * message of the last error on the calling thread is available from mx_last_error().
 * Calls from several host threads are safe: besides that thread-local string the library's only
 * mutable state is set-once caches (the per-device address of the static scratch of mx_gemm_static,
 * per-kernel "launch attribute set" flags and the CU count of the device that was current at the
 * first launch; a racing thread stores the same value).  The library serves one device model
 * (MI355X): with several GPUs in one process all of them are assumed to have the same CU count.
 * Nothing here allocates device memory: any workspace is passed in by the caller, except for
 * mx_gemm_static, whose scratch is a fixed buffer inside the library's device image.
 *
 * Each declaration names the reference interface (NVIDIA cuTile Python, path:line) it stands in for.
 */
#ifndef MXGEMM_H
#define MXGEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MXGEMM_VERSION 103

/* Exported symbols (the library is built with hidden default visibility). */
#if defined(__GNUC__)
#define MX_API __attribute__((visibility("default")))
#else
#define MX_API
#endif

/* Error codes. */
enum {
  MX_OK = 0,
  MX_ERR_INVALID = -1,      /* bad argument (null pointer, rank, negative stride ...)            */
  MX_ERR_SHAPE = -2,        /* shapes of operands / scales / output do not agree                 */
  MX_ERR_DTYPE = -3,        /* unsupported dtype or dtype combination                            */
  MX_ERR_LAYOUT = -4,       /* layout not supported by the requested kernel                      */
  MX_ERR_WORKSPACE = -5,    /* workspace missing or too small                                    */
  MX_ERR_DEVICE = -6,       /* no gfx950 device / HIP error                                      */
  MX_ERR_LAUNCH = -7        /* kernel launch failed                                              */
};

/* Element / scale / output type codes.  The three element formats use the codes the CDNA4
 * v_mfma_scale_f32_*_f8f6f4 instruction uses for its cbsz/blgp fields. */
enum {
  MX_E4M3 = 0,   /* float8_e4m3fn, 1 byte                                            */
  MX_E5M2 = 1,   /* float8_e5m2,   1 byte                                            */
  MX_E2M1 = 4,   /* float4_e2m1fn, two per byte, low nibble = even logical element   */
  MX_E8M0 = 8,   /* float8_e8m0fnu scale byte, value 2^(b-127), 0xFF = NaN           */
  MX_F32 = 16,
  MX_BF16 = 17,
  MX_F16 = 18,
  MX_I32 = 24
};

/*
 * Tensor descriptor: pointer + logical shape + strides.  Mirrors the per-array words the
 * reference's launcher passes to a kernel (ptr, shape[ndim], stride[ndim];
 * cext/tile_kernel.cpp:1883-1917, 1999-2002).
 *   shape[]  -- LOGICAL element counts (for MX_E2M1: number of 4-bit elements).
 *   stride[] -- in units of the storage type: bytes for all 8- and 4-bit formats, elements for
 *               f32/bf16/i32.  For MX_E2M1 exactly one dimension is the packed one: it has stride 1
 *               and holds two logical elements per byte; `packed_dim` names it.
 */
typedef struct mx_tensor {
  void* ptr;
  int32_t dtype;
  int32_t ndim;          /* 1..4 */
  int64_t shape[4];
  int64_t stride[4];
  int32_t packed_dim;    /* MX_E2M1 only: index of the dimension packed two-per-byte; else -1 */
  int32_t reserved;
} mx_tensor;

/* Scale tensor layouts accepted by mx_gemm / mx_gemm_grouped. */
enum {
  MX_SCALE_2D = 0,        /* logical [rows, K/B] (A) or [K/B, cols] (B), any strides
                             (samples/BlockScaledMatMul.py:243-250)                              */
  MX_SCALE_SWIZZLE_32_4_4 = 1, /* contiguous [rows/128, (K/B)/4, 32, 16] as produced by
                             swizzle_32_4_4 (test/kernels/kernel_utils.py:83-98); for B the rows
                             are the N index                                                      */
  MX_SCALE_NATIVE = 2,    /* this library's MFMA-ready layout written by mx_pack_scales for the
                             kernels on v_mfma_scale_f32_16x16x128_f8f6f4 (every MFMA kernel but the
                             two below); A and B scales are packed differently (MX_OPERAND_*)      */
  MX_SCALE_NATIVE32 = 3   /* the MFMA-ready layout of the kernels on v_mfma_scale_f32_32x32x64_f8f6f4
                             (MX_KERNEL_MFMA_PINGPONG32, MX_KERNEL_MFMA_W4_PERSISTENT)             */
};

/* Which operand of the product a native-layout scale tensor belongs to (mx_pack_scales). */
enum {
  MX_OPERAND_A = 0,
  MX_OPERAND_B = 1
};

/* Kernel selection. */
enum {
  MX_KERNEL_AUTO = 0,
  MX_KERNEL_GENERIC = 1,      /* one thread per output element; any strides / packing / block  */
  MX_KERNEL_MFMA_128x128 = 2, /* v_mfma_scale tiles, 128x128 macro tile, 4 waves                */
  MX_KERNEL_MFMA_256x256 = 3, /* 256x256 macro tile, 8 waves                                    */
  MX_KERNEL_MFMA_256x256_W4 = 4, /* 256x256 macro tile, 4 waves                                 */
  MX_KERNEL_DECODE = 5,       /* skinny-M weight-streaming kernel: 8-bit activations x FP4 weights,
                                 K % 512 == 0, N % 16 == 0; 32 rows of A and 8192 of K per launch, more
                                 rows (up to 128; MX_KERNEL_AUTO: up to 64) in slabs, a longer K in chunks
                                 summed in fp32 in the workspace                                  */
  MX_KERNEL_MFMA_PINGPONG = 6, /* 256x256 macro tile, two 4-wave teams alternating LDS/MFMA phases,
                                 v_mfma_scale_f32_16x16x128_f8f6f4                                */
  MX_KERNEL_MFMA_PINGPONG32 = 7, /* the same schedule on v_mfma_scale_f32_32x32x64_f8f6f4; 8-bit
                                 element formats only                                             */
  MX_KERNEL_MFMA_W4_PERSISTENT = 8 /* 256x256 macro tile, four waves of 128x128 (one per SIMD, 512
                                 registers), self-pipelined, 32x32x64 instruction; plain products of
                                 8-bit operands with K >= 384                                     */
};

typedef struct mx_gemm_opts {
  int32_t struct_size;    /* sizeof(mx_gemm_opts), for forward compatibility                    */
  int32_t accumulate;     /* 0: C = A@B ; 1: C = A@B + C  (the `acc` operand of ct.mma_scaled)   */
  int32_t a_scale_layout; /* MX_SCALE_*                                                          */
  int32_t b_scale_layout;
  int32_t kernel;         /* MX_KERNEL_*                                                         */
  int32_t block_size;     /* scaling block size B along K: 32 (16 only with MX_KERNEL_GENERIC)   */
  int32_t split_k;        /* mx_gemm only: 0 = the library decides, 1 = never split K, n > 1 = n K-slices
                             (K must be a multiple of 512 n; plain 2-D scale layouts; one-tile MFMA
                             kernels).  Slices run side by side and a second kernel adds their fp32
                             partial products in a fixed order: the split-K scheme of
                             matmul_split_k_kernel, test/kernels/matmul.py:103-140, for small M x N
                             with a long K                                                        */
  int32_t reserved;
} mx_gemm_opts;

/* Library version (MXGEMM_VERSION of the built library). */
MX_API int mx_version(void);

/* Message of the last error raised on the calling thread ("" if none).
 * Stands in for the Python exception text of cext/tile_kernel.cpp:3910-3916. */
MX_API const char* mx_last_error(void);

/* Returns 0 if the current HIP device is a gfx950 part, MX_ERR_DEVICE otherwise.
 * (reference: get_compute_capability gate, samples/BlockScaledMatMul.py:308-311.) */
MX_API int mx_device_check(void);

/*
 * Bytes of device workspace mx_gemm needs for the given problem (native re-layout of the scale
 * tensors, split-K partial products, the fp32 chunk sums of the skinny-M kernel for K > 8192).  0 if both
 * scale tensors are already in a native layout and nothing else is needed, or the generic kernel is used.
 */
MX_API int64_t mx_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, const mx_gemm_opts* opts);

/*
 * C[M,N] (+)= sum_k A[m,k]*As[m,k/B] * B[k,n]*Bs[k/B,n]   with fp32 accumulation.
 * Replaces: ct.launch(stream, grid, block_scaled_matmul_kernel, (A, A_scale, B, B_scale, C, tm, tn,
 * tk, scaling_block_size))  -- samples/BlockScaledMatMul.py:294-295, kernel
 * test/kernels/scaled_matmul.py:12-114, op semantics src/cuda/tile/_stub.py:2198-2235.
 *   A  [M,K]  MX_E4M3 | MX_E5M2 | MX_E2M1        As [M,K/B] MX_E8M0 (or 4-D swizzled / native)
 *   B  [K,N]  same family (formats may differ)    Bs [K/B,N]
 *   C  [M,N]  MX_F32 | MX_BF16
 * The MFMA kernels need K-contiguous A (stride[1]==1) and B (stride[0]==1), 16-byte aligned rows
 * and block_size 32; MX_KERNEL_AUTO falls back to the generic kernel otherwise.
 * Optional leading batch dimension (ndim 3, test/test_mma_scaled.py:128-145): one 2-D product per batch
 * entry on the same kernels, batches of size 1 broadcast; the entries share the workspace in stream order.
 */
MX_API int mx_gemm(const mx_tensor* A, const mx_tensor* A_scale, const mx_tensor* B,
            const mx_tensor* B_scale, mx_tensor* C, const mx_gemm_opts* opts, void* workspace,
            int64_t workspace_bytes, void* stream);

/*
 * mx_gemm for callers that cannot allocate or hand over device scratch: code running under HIP-graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its launcher needs no
 * scratch; cext/tile_kernel.cpp:3874-3919 only launches).  Same operands, options, results and errors as
 * mx_gemm, without the workspace arguments: the scale re-layout (and the split-K partial products) go to a
 * buffer of MX_STATIC_SCRATCH_BYTES inside the library's own device image, one per GPU, held until the process
 * ends.  Calls no hipMalloc / hipFree or any allocating routine.  A problem whose mx_gemm_workspace_bytes()
 * exceeds MX_STATIC_SCRATCH_BYTES is refused with MX_ERR_WORKSPACE (8 MiB covers M*K + N*K <= 128 Mi elements,
 * e.g. 16384 x 16384 x 4096; use mx_gemm beyond that).  Every call on a GPU shares that GPU's buffer, which
 * keeps the previous call's contents; nothing in it has to start at zero (each call rewrites all it reads).
 * Calls on one stream are ordered; calls that overlap on one GPU (several streams or host threads) race.
 * The buffer's address is resolved on the first call on a device, or by mx_device_check(): make one of the
 * two, and one warm-up call per kernel, before a capture begins.
 */
#define MX_STATIC_SCRATCH_BYTES (8 * 1024 * 1024)
MX_API int64_t mx_static_scratch_bytes(void);
MX_API int mx_gemm_static(const mx_tensor* A, const mx_tensor* A_scale, const mx_tensor* B,
                   const mx_tensor* B_scale, mx_tensor* C, const mx_gemm_opts* opts, void* stream);

/*
 * A list of independent block-scaled products C[i] = A[i] x B[i] (problem sizes may all differ), the
 * block-scaled counterpart of grouped_matmul_kernel(As, Bs, Cs, ...), test/kernels/group_gemm.py:10-38.
 * The descriptor arrays hold `count` entries each; every problem follows the rules of mx_gemm.  All problems are
 * validated first: on error the index of the failing problem is part of mx_last_error().  A problem that is
 * refused by these checks (descriptors, shapes, dtypes, layouts, workspace) leaves nothing enqueued; a problem of the
 * kinds listed below as "the others" can still be refused by the kernel it is sent to (for example a forced kernel
 * that does not take its shape), after the problems in front of it have been enqueued.  The C tensors of a list must
 * not overlap: its problems run side by side, not in list order.  Problems that mx_gemm would give to its 128 x 128 one-tile kernel (the small and medium ones, which
 * is what such lists hold) run the way the reference's kernel does: one launch re-lays up to 64 scale
 * tensors, and one launch of persistent workgroups walks the concatenated tile list of up to 32 problems of one
 * element-format pair and output type (tile_idx += number of workgroups).  The others (large problems for the
 * persistent 256 x 256 kernel, skinny ones for the decode kernel, split-K, layouts of the general kernel) get a
 * call of their own behind them.  No host synchronisation.  The workspace holds one slice per problem
 * (mx_gemm_list_workspace_bytes is the sum of the single needs): the problems run side by side.  Empty problems
 * (M or N zero) are skipped.
 */
MX_API int64_t mx_gemm_list_workspace_bytes(int32_t count, const mx_tensor* A, const mx_tensor* B,
                                     const mx_gemm_opts* opts);
MX_API int mx_gemm_list(int32_t count, const mx_tensor* A, const mx_tensor* A_scale, const mx_tensor* B,
                 const mx_tensor* B_scale, mx_tensor* C, const mx_gemm_opts* opts, void* workspace,
                 int64_t workspace_bytes, void* stream);

/*
 * Timing aid, the counterpart of the reference launcher's _benchmark (cext/tile_kernel.cpp:3921-4042, used by
 * the tuner, src/cuda/tile/tune/_tune.py:339-395): `warmup` untimed mx_gemm calls, then `iters` calls, each
 * between its own pair of HIP events recorded on `stream`; times_ms[i] (host memory, `iters` floats) receives the
 * duration of call i, which includes whatever mx_gemm enqueues for it (scale re-layout unless the scales are
 * MX_SCALE_NATIVE).  Where the reference defeats the cache by writing an L2-sized buffer before each timed
 * launch, this rotates operand sets: the descriptor arrays hold `nsets` entries each and call i uses set
 * i % nsets, so give it enough distinct sets to exceed the 256 MiB Infinity Cache.  The only entry point that
 * synchronises: it returns after `stream` has drained.  Creates HIP events; allocates no device memory.
 */
MX_API int mx_bench_gemm(int32_t nsets, const mx_tensor* A, const mx_tensor* A_scale, const mx_tensor* B,
                  const mx_tensor* B_scale, mx_tensor* C, const mx_gemm_opts* opts, void* workspace,
                  int64_t workspace_bytes, int32_t warmup, int32_t iters, float* times_ms, void* stream);

/*
 * Grouped (MoE) variant.  Replaces: ct.launch(..., fused_moe_kernel, (A, B, C, topk_weights,
 * sorted_token_ids, sorted_expert_ids, num_token_replicas, mul_routed_weight, TILE_M, TILE_N,
 * TILE_K)) -- samples/MoE.py:338-375, kernel test/kernels/fused_moe.py:14-82, with the bf16 ct.mma
 * replaced by the block-scaled product.
 *   A  [T,K] tokens, As [T,K/32];  W [E,N,K] (K contiguous), Ws [E,N,K/32];  C [T*replicas? ,N]:
 *   for every slot p of sorted_token_ids with id = sorted_token_ids[p] < num_valid_ids:
 *       C[id,:] = (A[id / num_token_replicas,:] * As) @ (W[e,:,:] * Ws[e]).T * (w ? w[id] : 1)
 *   where e = sorted_expert_ids[p / tile_m] (an entry outside [0, E) is clamped into that range, so nothing
 *   outside W is ever read; its rows are unspecified).  Slots holding the sentinel are skipped, wherever they
 *   sit in a tile.
 *   topk_weights may be NULL (no routed-weight multiply).
 * Workspace: mx_gemm_grouped_workspace_bytes().
 */
MX_API int64_t mx_gemm_grouped_workspace_bytes(int64_t num_slots, int64_t N, int64_t K, int64_t E,
                                        const mx_gemm_opts* opts);
MX_API int mx_gemm_grouped(const mx_tensor* A, const mx_tensor* A_scale, const mx_tensor* W,
                    const mx_tensor* W_scale, mx_tensor* C, const float* topk_weights,
                    const int32_t* sorted_token_ids, int64_t num_slots,
                    const int32_t* sorted_expert_ids, int32_t tile_m, int32_t num_token_replicas,
                    int64_t num_valid_ids, const mx_gemm_opts* opts, void* workspace,
                    int64_t workspace_bytes, void* stream);

/*
 * Device-side replacement of moe_align_tile_size_torch (test/kernels/fused_moe.py:113-173): stable
 * counting sort of the flattened expert ids, each expert padded to a multiple of tile_m with the
 * sentinel value num_ids.  Outputs must hold mx_moe_align_max_slots(num_ids, num_experts, tile_m)
 * int32 slots and that number / tile_m blocks; unused trailing slots are filled with the sentinel
 * and unused trailing blocks with expert 0.  *num_slots_out (device int32, optional) receives the
 * number of slots actually used.  No host synchronisation, no atomics on global memory, every output
 * element written exactly once.
 */
MX_API int64_t mx_moe_align_max_slots(int64_t num_ids, int32_t num_experts, int32_t tile_m);
/* Scratch for the per-chunk histograms of mx_moe_align: 0 for up to 1024 ids (one workgroup), otherwise
 * chunks x num_experts int32 (the ids are sorted by up to 256 workgroups, more beyond 16.7 M ids). */
MX_API int64_t mx_moe_align_workspace_bytes(int64_t num_ids, int32_t num_experts);
MX_API int mx_moe_align(const int32_t* topk_ids, int64_t num_ids, int32_t num_experts, int32_t tile_m,
                 int32_t* sorted_token_ids, int32_t* sorted_expert_ids, int32_t* num_slots_out,
                 void* workspace, int64_t workspace_bytes, void* stream);

/*
 * MX quantisation of the last axis in blocks of 32 (replaces the torch-op sequence of
 * block_quantize, test/kernels/kernel_utils.py:38-80).
 *   x      [rows, K] MX_F32 | MX_BF16 | MX_F16, last stride 1
 *   xq     [rows, Kpad] MX_E4M3 | MX_E5M2 (1 byte each) or MX_E2M1 (packed along K), Kpad = K
 *          rounded up to 32 (tail zero-padded as the reference does)
 *   scale  [rows, Kpad/32] MX_E8M0
 *   scale_mode 0 = "ceil":  2^ceil(log2(max(amax/448, 1e-12))), non-saturating element cast
 *              1 = "floor": 2^(floor(log2 amax) - emax_elem), saturating element cast (OCP MX v1.0)
 */
MX_API int mx_quantize(const mx_tensor* x, mx_tensor* xq, mx_tensor* scale, int32_t scale_mode,
                void* stream);

/*
 * Fused activation producer of the MoE pipeline: silu(gate) * up, MX-quantised in one pass (replaces
 * silu_and_mul_kernel, test/kernels/fused_moe.py:85-108, followed by block_quantize, so that the
 * down-projection of cutile_moe, samples/MoE.py:197-288, can also run block-scaled).
 *   gate_up [rows, 2F] MX_F32 | MX_BF16 | MX_F16, last stride 1: gate = [:, :F], up = [:, F:]
 *   xq      [rows, Fpad] elements, scale [rows, Fpad/32] MX_E8M0, scale_mode: as mx_quantize
 * The product is formed in fp32 as a fixed sequence of correctly rounded operations
 * (a / (1 + 2^(-a log2 e)) * b with a degree-7 polynomial for the fractional power), so a host
 * restatement reproduces it bit for bit; it is within a few 1e-7 relative of torch's silu(a) * b.
 */
MX_API int mx_silu_mul_quantize(const mx_tensor* gate_up, mx_tensor* xq, mx_tensor* scale, int32_t scale_mode,
                         void* stream);

/*
 * Re-lays a scale tensor into an MFMA-ready native layout consumed by the MFMA kernels
 * (no reference counterpart: the reference's swizzle_32_4_4, test/kernels/kernel_utils.py:83-98,
 * is the Blackwell analogue).  `scale` is [rows, K/32] logical with any strides (MX_SCALE_2D; pass a
 * transposed descriptor for a [K/32, cols] tensor), or the contiguous 4-D swizzled tensor
 * (MX_SCALE_SWIZZLE_32_4_4); an optional leading batch dimension (experts) is kept.
 * `native_layout` is MX_SCALE_NATIVE or MX_SCALE_NATIVE32 (the kernels that will read it), `operand`
 * MX_OPERAND_A (activations / left operand) or MX_OPERAND_B (weights / right operand, also the expert
 * weights of mx_gemm_grouped): MX_SCALE_NATIVE orders the B rows the way the kernels feed them to the
 * instruction, so a tensor packed for one operand must not be passed as the other.
 * `packed` must hold mx_packed_scale_bytes(rows, K) bytes per batch entry (the same for every layout).
 */
MX_API int64_t mx_packed_scale_bytes(int64_t rows, int64_t K);
MX_API int mx_pack_scales(const mx_tensor* scale, int32_t layout, int64_t rows, int64_t K, int32_t native_layout,
                   int32_t operand, void* packed, void* stream);

/*
 * Measurement aid (no reference counterpart; the reference measures whole kernels only, cext/tile_kernel.cpp:3921-4042):
 * the rate at which the chip runs v_mfma_scale_f32_16x16x128_f8f6f4 out of registers alone on the given operand bits
 * -- no LDS, no memory traffic -- i.e. the ceiling that the data itself (through the chip's power management) puts
 * on any GEMM schedule.  `workgroups` workgroups of 8 waves (two per SIMD, one workgroup per CU when workgroups =
 * the CU count) each load 8 + 4 operand fragments per wave from `frags` (12 x 512 fragments of 32 bytes, [fragment]
 * [thread]; MX_E2M1 uses the first 16 bytes of each; unit scales) and multiply all 32 pairs `iters` times:
 * workgroups x 8 x iters x 32 x 65536 flop per launch.  sink[workgroups x 512] receives a value that keeps the
 * products alive.  Asynchronous on `stream`; time it with events, and take the clock it ran at from the
 * SQ_BUSY_CYCLES counter of a profiler run over the launch's duration.
 */
MX_API int mx_probe_mfma_rate(int32_t fmt, const void* frags, int32_t workgroups, int32_t iters, float* sink,
                       void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MXGEMM_H */
