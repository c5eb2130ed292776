// C ABI of libmxgemm.so: argument validation and kernel dispatch.  See include/mxgemm.h.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <vector>

#include "mx_common.h"

// Scratch of mx_gemm_static: lives in the library's device image, one copy per GPU the library runs on, held
// until the process ends.  Host code never uses this name as an address: static_scratch() below resolves the
// device address once per device with hipGetSymbolAddress and everything else uses that pointer.
static __device__ __align__(256) unsigned char scratch[MX_STATIC_SCRATCH_BYTES];

namespace mx {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

namespace {

inline bool is_elem(int d) { return d == MX_E4M3 || d == MX_E5M2 || d == MX_E2M1; }
inline int64_t round256(int64_t b) { return (b + 255) & ~(int64_t)255; }

// kernel MX_KERNEL_AUTO uses for large problems
constexpr int big_tile_kernel() { return MX_KERNEL_MFMA_PINGPONG; }

// Problems MX_KERNEL_AUTO gives to the persistent 256x256 kernel: enough 256x256 tiles to occupy most of the
// 256 CUs (measured crossover against the 128x128 one-tile kernel, which has four times as many workgroups
// to spread: 128 tiles -> 128x128 is 14 % faster, 144 tiles -> 256x256 is 26 % faster).
inline bool big_tile_problem(int64_t M, int64_t N) {
  return M > 128 && N > 128 && ((M + 255) / 256) * ((N + 255) / 256) >= 144;
}

// native scale layout a kernel reads: the two kernels on the 32x32x64 instruction have their own
inline int native_layout_of(int kernel) {
  return (kernel == MX_KERNEL_MFMA_PINGPONG32 || kernel == MX_KERNEL_MFMA_W4_PERSISTENT) ? MX_SCALE_NATIVE32
                                                                                       : MX_SCALE_NATIVE;
}
inline bool is_native(int layout) { return layout == MX_SCALE_NATIVE || layout == MX_SCALE_NATIVE32; }

// The decode kernel takes K up to kDecodeChunk per launch; a longer K runs as one launch per chunk, the chunks adding
// up in an fp32 buffer of the workspace that a last pass converts into C.
constexpr int64_t kDecodeChunk = 8192;
// One launch of it multiplies up to 32 rows of X; more rows run slab by slab, each slab streaming the weights again
// (the second pass finds most of a weight matrix of up to 256 MiB in the Infinity Cache).  MX_KERNEL_AUTO does that
// up to kDecodeAutoM rows (measured on 28672 x 8192 FP4 weights: M = 64 takes 2 x 26 us this way against 62 us on the
// tiled kernel, whose time hardly grows up to M = 128); an explicit MX_KERNEL_DECODE up to kDecodeMaxM.
constexpr int64_t kDecodeAutoM = 64, kDecodeMaxM = 128;
inline bool decode_shape(int64_t M, int64_t N, int64_t K) {
  return M >= 1 && M <= kDecodeMaxM && K % 512 == 0 && N % 16 == 0;
}
// workspace of that buffer; depends on (M, N, K, opts) only, so it is also counted for problems whose operand types
// then send them to another kernel
inline int64_t decode_partial_bytes(int64_t M, int64_t N, int64_t K, const mx_gemm_opts& o) {
  if ((o.kernel != MX_KERNEL_AUTO && o.kernel != MX_KERNEL_DECODE) || !decode_shape(M, N, K) || K <= kDecodeChunk)
    return 0;
  return round256(M * N * 4);
}

const mx_gemm_opts kDefaultOpts = {sizeof(mx_gemm_opts), 0, MX_SCALE_2D, MX_SCALE_2D, MX_KERNEL_AUTO, 32, 0, 0};

// Number of K-slices for a problem that ends up on a one-tile MFMA kernel (1 = no split).  Depends only on
// (M, N, K, opts) so that mx_gemm_workspace_bytes and mx_gemm agree.  Automatic rule: split when the tiles
// of the 128x128 kernel cover less than half of the CUs and every slice keeps at least two K-quads.
int plan_k_splits(int64_t M, int64_t N, int64_t K, const mx_gemm_opts& o) {
  if (o.split_k == 1 || o.a_scale_layout != MX_SCALE_2D || o.b_scale_layout != MX_SCALE_2D || o.block_size != 32)
    return 1;
  if (o.kernel != MX_KERNEL_AUTO && o.kernel != MX_KERNEL_MFMA_128x128 && o.kernel != MX_KERNEL_MFMA_256x256 &&
      o.kernel != MX_KERNEL_MFMA_256x256_W4)
    return 1;
  if (K <= 0 || K % 512 != 0 || M <= 0 || N <= 0) return 1;
  if (o.split_k > 1) return (K % ((int64_t)512 * o.split_k) == 0) ? o.split_k : -1;   // -1: cannot honour
  if (o.kernel != MX_KERNEL_AUTO && o.kernel != MX_KERNEL_MFMA_128x128) return 1;
  if (o.kernel == MX_KERNEL_AUTO && big_tile_problem(M, N)) return 1;   // big-tile kernel
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  if (tiles * 2 > 256 || K < 2048) return 1;
  int64_t s = 256 / tiles;
  if (s > K / 1024) s = K / 1024;
  while (s > 1 && K % (512 * s) != 0) --s;
  return (int)(s < 1 ? 1 : s);
}


int check_tensor(const mx_tensor* t, const char* name, int min_nd, int max_nd) {
  if (!t) return set_error(MX_ERR_INVALID, "%s: null descriptor", name);
  if (t->ndim < min_nd || t->ndim > max_nd)
    return set_error(MX_ERR_SHAPE, "%s: expected %d..%d dimensions, got %d", name, min_nd, max_nd, t->ndim);
  int64_t numel = 1;
  for (int i = 0; i < t->ndim; ++i) {
    if (t->shape[i] < 0) return set_error(MX_ERR_SHAPE, "%s: negative extent", name);
    if (t->stride[i] < 0) return set_error(MX_ERR_LAYOUT, "%s: negative strides are not supported", name);
    numel *= t->shape[i];
  }
  if (numel > 0 && !t->ptr) return set_error(MX_ERR_INVALID, "%s: null data pointer", name);
  return MX_OK;
}

bool pair_supported_by_mfma(int a, int b) {
  return (a == MX_E4M3 && b == MX_E4M3) || (a == MX_E5M2 && b == MX_E5M2) ||
         (a == MX_E2M1 && b == MX_E2M1) || (a == MX_E4M3 && b == MX_E2M1);
}

// Checks the layout preconditions of the MFMA kernels for a K-contiguous operand with `rows` rows.
// Returns nullptr if fine, otherwise the reason.
const char* mfma_operand_issue(const void* ptr, int64_t rows, int64_t ld_bytes, int64_t k_stride,
                               int fmt, int packed_ok) {
  if (k_stride != 1) return "K axis is not contiguous";
  if (fmt == MX_E2M1 && !packed_ok) return "FP4 operand is not packed along K";
  if (((uintptr_t)ptr) % 16 != 0) return "base pointer is not 16-byte aligned";
  if (ld_bytes % 16 != 0) return "row pitch is not a multiple of 16 bytes";
  if (rows * ld_bytes >= ((int64_t)1 << 31)) return "operand spans 2 GiB or more";
  return nullptr;
}

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device (each GPU holds its own copy at its own address)
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(MX_ERR_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return set_error(MX_ERR_DEVICE, "device index %d out of range", dev);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return set_error(MX_ERR_DEVICE, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // a racing thread stores the same address
  }
  *out = p;
  return MX_OK;
}
}  // namespace
}  // namespace mx

using namespace mx;

extern "C" {

int mx_version(void) { return MXGEMM_VERSION; }

const char* mx_last_error(void) { return g_err; }

int mx_device_check(void) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(MX_ERR_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return set_error(MX_ERR_DEVICE, "hipGetDeviceProperties: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(MX_ERR_DEVICE, "libmxgemm is built for gfx950 only, device is %s", prop.gcnArchName);
  void* p = nullptr;
  return static_scratch(&p);   // set-up of mx_gemm_static on this device
}

int64_t mx_packed_scale_bytes(int64_t rows, int64_t K) {
  return round256(packed_scale_dwords(rows, K) * 4);
}

int64_t mx_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, const mx_gemm_opts* opts) {
  const mx_gemm_opts& o = opts ? *opts : kDefaultOpts;
  if (o.kernel == MX_KERNEL_GENERIC) return 0;
  if (o.kernel == MX_KERNEL_DECODE) return decode_partial_bytes(M, N, K, o);
  int64_t b = decode_partial_bytes(M, N, K, o);
  const int S = plan_k_splits(M, N, K, o);
  if (S > 1) {   // per-slice packed scales and the fp32 partial products
    b += S * (mx_packed_scale_bytes(M, K / S) + mx_packed_scale_bytes(N, K / S));
    b += round256(S * M * N * 4);
    return b;
  }
  if (!is_native(o.a_scale_layout)) b += mx_packed_scale_bytes(M, K);
  if (!is_native(o.b_scale_layout)) b += mx_packed_scale_bytes(N, K);
  return b;
}

int64_t mx_gemm_grouped_workspace_bytes(int64_t num_slots, int64_t N, int64_t K, int64_t E,
                                        const mx_gemm_opts* opts) {
  const mx_gemm_opts& o = opts ? *opts : kDefaultOpts;
  if (o.kernel == MX_KERNEL_GENERIC) return 0;
  int64_t b = mx_packed_scale_bytes(num_slots, K);
  if (!is_native(o.b_scale_layout)) b += E * mx_packed_scale_bytes(N, K);
  return b;
}

namespace {
// a 4-D swizzle_32_4_4 scale tensor must be the contiguous [rows / 128, (K / 32) / 4, 32, 16] array
int check_swizzled_scale(const mx_tensor* scale, const char* name, int64_t rows, int64_t KB) {
  if (scale->ndim != 4 || scale->shape[2] != 32 || scale->shape[3] != 16)
    return set_error(MX_ERR_SHAPE, "%s: swizzled scale layout expects [rows/128, K/128, 32, 16]", name);
  if (rows % 128 != 0 || KB % 4 != 0 || scale->shape[0] != rows / 128 || scale->shape[1] != KB / 4)
    return set_error(MX_ERR_SHAPE, "%s: swizzled scale shape does not match rows=%lld, K blocks=%lld (rows %% 128 "
                     "and blocks %% 4 must be 0)", name, (long long)rows, (long long)KB);
  if (scale->stride[3] != 1 || scale->stride[2] != 16 || scale->stride[1] != 512 ||
      scale->stride[0] != 512 * (KB / 4))
    return set_error(MX_ERR_LAYOUT, "%s: swizzled scale tensor must be contiguous", name);
  return MX_OK;
}

// validates a scale tensor against (rows, K) and describes its re-layout into `packed`
int make_pack_args(const mx_tensor* scale, int32_t layout, int64_t rows, int64_t K, void* packed, int target,
                   PackArgs& p) {
  if (int rc = check_tensor(scale, "scale", 2, 4)) return rc;
  if (!packed) return set_error(MX_ERR_INVALID, "packed: null pointer");
  if (K % 32 != 0) return set_error(MX_ERR_SHAPE, "K (%lld) must be a multiple of 32", (long long)K);
  if (((uintptr_t)packed) % 16 != 0) return set_error(MX_ERR_LAYOUT, "packed buffer must be 16-byte aligned");
  p = PackArgs{};
  p.src = (const uint8_t*)scale->ptr;
  p.dst = (uint32_t*)packed;
  p.rows = rows;
  p.K = K;
  p.layout = layout;
  p.target = target;
  p.batch = 1;
  p.replicas = 1;
  const int64_t KB = K / 32;
  if (layout == MX_SCALE_2D) {
    const int nd = scale->ndim;
    if (nd != 2 && nd != 3) return set_error(MX_ERR_SHAPE, "2-D scale layout expects [rows, K/32] with an optional batch");
    if (scale->shape[nd - 2] != rows || scale->shape[nd - 1] != KB)
      return set_error(MX_ERR_SHAPE, "scale shape (%lld, %lld) does not match rows=%lld, K/32=%lld",
                       (long long)scale->shape[nd - 2], (long long)scale->shape[nd - 1], (long long)rows,
                       (long long)KB);
    p.s_row = scale->stride[nd - 2];
    p.s_kb = scale->stride[nd - 1];
    if (nd == 3) {
      p.batch = (int32_t)scale->shape[0];
      p.s_batch = scale->stride[0];
    }
  } else if (layout == MX_SCALE_SWIZZLE_32_4_4) {
    if (int rc = check_swizzled_scale(scale, "scale", rows, KB)) return rc;
  } else {
    return set_error(MX_ERR_INVALID, "mx_pack_scales: unknown source layout %d", layout);
  }
  return MX_OK;
}
}  // namespace

int mx_pack_scales(const mx_tensor* scale, int32_t layout, int64_t rows, int64_t K, int32_t native_layout,
                   int32_t operand, void* packed, void* stream) {
  if (!is_native(native_layout))
    return set_error(MX_ERR_INVALID, "mx_pack_scales: native_layout must be MX_SCALE_NATIVE or MX_SCALE_NATIVE32");
  if (operand != MX_OPERAND_A && operand != MX_OPERAND_B)
    return set_error(MX_ERR_INVALID, "mx_pack_scales: operand must be MX_OPERAND_A or MX_OPERAND_B");
  const int target = native_layout == MX_SCALE_NATIVE32 ? kPackTile32 : (operand == MX_OPERAND_B ? kPackB : kPackA);
  PackArgs p;
  if (int rc = make_pack_args(scale, layout, rows, K, packed, target, p)) return rc;
  return launch_pack_scales(p, (hipStream_t)stream);
}

namespace {
// What mx_gemm would launch for a problem that ends on the 128 x 128 one-tile kernel without split-K: the list
// entry point collects these and runs them as one batched scale re-layout and one persistent GEMM launch.
struct GemmPlan {
  GemmArgs g;
  PackArgs pa, pb;
  bool pack_a, pack_b;
};
constexpr int kPlanNotSimple = 1;   // gemm_impl with a plan: the problem needs its own mx_gemm call

int gemm_impl(const mx_tensor* A, const mx_tensor* As, const mx_tensor* B, const mx_tensor* Bs, mx_tensor* C,
              const mx_gemm_opts* opts, void* workspace, int64_t workspace_bytes, void* stream, GemmPlan* plan);
}  // namespace

int mx_gemm(const mx_tensor* A, const mx_tensor* As, const mx_tensor* B, const mx_tensor* Bs, mx_tensor* C,
            const mx_gemm_opts* opts, void* workspace, int64_t workspace_bytes, void* stream) {
  return gemm_impl(A, As, B, Bs, C, opts, workspace, workspace_bytes, stream, nullptr);
}

namespace {
// mx_gemm; with `plan` nothing is launched: a problem of the simple kind is described in *plan (return MX_OK),
// any other valid problem returns kPlanNotSimple
int gemm_impl(const mx_tensor* A, const mx_tensor* As, const mx_tensor* B, const mx_tensor* Bs, mx_tensor* C,
              const mx_gemm_opts* opts, void* workspace, int64_t workspace_bytes, void* stream, GemmPlan* plan) {
  const mx_gemm_opts& o = opts ? *opts : kDefaultOpts;
  if (int rc = check_tensor(A, "A", 2, 3)) return rc;
  if (int rc = check_tensor(B, "B", 2, 3)) return rc;
  if (int rc = check_tensor(As, "A_scale", 2, 4)) return rc;
  if (int rc = check_tensor(Bs, "B_scale", 2, 4)) return rc;
  if (int rc = check_tensor(C, "C", 2, 3)) return rc;
  if (!is_elem(A->dtype) || !is_elem(B->dtype))
    return set_error(MX_ERR_DTYPE, "A/B must be MX_E4M3, MX_E5M2 or MX_E2M1 (got %d, %d)", A->dtype, B->dtype);
  if (C->dtype != MX_F32 && C->dtype != MX_BF16)
    return set_error(MX_ERR_DTYPE, "C must be MX_F32 or MX_BF16 (got %d)", C->dtype);
  if (As->dtype != Bs->dtype) return set_error(MX_ERR_DTYPE, "A_scale and B_scale must have the same dtype");
  if (As->dtype != MX_E8M0 && As->dtype != MX_E4M3)
    return set_error(MX_ERR_DTYPE, "scale dtype must be MX_E8M0 (or MX_E4M3 for FP4 with block 16)");
  if (o.block_size != 32 && o.block_size != 16)
    return set_error(MX_ERR_INVALID, "block_size must be 16 or 32 (got %d)", o.block_size);

  const int and_ = A->ndim, bnd = B->ndim, cnd = C->ndim;
  const int64_t M = A->shape[and_ - 2], K = A->shape[and_ - 1];
  const int64_t Kb = B->shape[bnd - 2], N = B->shape[bnd - 1];
  if (K != Kb)
    return set_error(MX_ERR_SHAPE, "Incompatible matrices: K dimension of A (%lld) must match K dimension of B (%lld)",
                     (long long)K, (long long)Kb);
  if (K % o.block_size != 0)
    return set_error(MX_ERR_SHAPE, "K (%lld) must be a multiple of the scaling block size %d", (long long)K,
                     o.block_size);
  const int64_t batchA = and_ == 3 ? A->shape[0] : 1, batchB = bnd == 3 ? B->shape[0] : 1;
  if (batchA != batchB && batchA != 1 && batchB != 1)
    return set_error(MX_ERR_SHAPE, "batch dimensions %lld and %lld cannot be broadcast", (long long)batchA,
                     (long long)batchB);
  const int64_t batch = batchA > batchB ? batchA : batchB;
  const bool batched = and_ == 3 || bnd == 3;
  if ((batched && (cnd != 3 || C->shape[0] != batch)) || (!batched && cnd != 2) || C->shape[cnd - 2] != M ||
      C->shape[cnd - 1] != N)
    return set_error(MX_ERR_SHAPE, "C has the wrong shape for a (%lld x %lld x %lld) product", (long long)M,
                     (long long)N, (long long)K);
  if (A->dtype == MX_E2M1 && A->packed_dim != and_ - 1 && A->packed_dim != and_ - 2)
    return set_error(MX_ERR_LAYOUT, "A: packed_dim must name the M or K dimension");
  if (B->dtype == MX_E2M1 && B->packed_dim != bnd - 1 && B->packed_dim != bnd - 2)
    return set_error(MX_ERR_LAYOUT, "B: packed_dim must name the K or N dimension");
  const int64_t KB = K / o.block_size;

  // ---- scale shapes --------------------------------------------------------------------------------
  if (o.a_scale_layout == MX_SCALE_2D) {
    const int nd = As->ndim;
    if (nd != and_ || As->shape[nd - 2] != M || As->shape[nd - 1] != KB || (nd == 3 && As->shape[0] != batchA))
      return set_error(MX_ERR_SHAPE, "A_scale shape is not compatible with A: expected [.., %lld, %lld]",
                       (long long)M, (long long)KB);
  }
  if (o.b_scale_layout == MX_SCALE_2D) {
    const int nd = Bs->ndim;
    if (nd != bnd || Bs->shape[nd - 2] != KB || Bs->shape[nd - 1] != N || (nd == 3 && Bs->shape[0] != batchB))
      return set_error(MX_ERR_SHAPE, "B_scale shape is not compatible with B: expected [.., %lld, %lld]",
                       (long long)KB, (long long)N);
  }
  if (M == 0 || N == 0) return plan ? kPlanNotSimple : MX_OK;

  // ---- batched operands (test/test_mma_scaled.py:128-145): one 2-D product per batch entry, size-1
  // batches broadcast; stream order lets the entries share the workspace.  Layouts only the generic
  // kernel reads (block 16, E4M3 scales) keep its own batched launch. --------------------------------
  if (batched && o.kernel != MX_KERNEL_GENERIC && o.block_size == 32 && As->dtype == MX_E8M0 &&
      o.a_scale_layout == MX_SCALE_2D && o.b_scale_layout == MX_SCALE_2D) {
    if (plan) return kPlanNotSimple;
    auto slice = [](const mx_tensor* t, int64_t b, int elem_bytes) {
      mx_tensor v = *t;
      if (t->ndim == 3) {
        v.ptr = (uint8_t*)t->ptr + (t->shape[0] > 1 ? b : 0) * t->stride[0] * elem_bytes;
        v.ndim = 2;
        for (int i = 0; i < 2; ++i) { v.shape[i] = t->shape[i + 1]; v.stride[i] = t->stride[i + 1]; }
        if (v.packed_dim >= 0) v.packed_dim -= 1;
      }
      return v;
    };
    const int c_bytes = C->dtype == MX_BF16 ? 2 : 4;
    for (int64_t b = 0; b < batch; ++b) {
      const mx_tensor a2 = slice(A, b, 1), as2 = slice(As, b, 1), b2 = slice(B, b, 1), bs2 = slice(Bs, b, 1);
      mx_tensor c2 = slice(C, b, c_bytes);
      if (int rc = mx_gemm(&a2, &as2, &b2, &bs2, &c2, &o, workspace, workspace_bytes, stream)) return rc;
    }
    return MX_OK;
  }

  // ---- can the MFMA path take it? ------------------------------------------------------------------
  const char* why = nullptr;
  const int64_t a_ld = A->stride[and_ - 2], b_ld = B->stride[bnd - 1];
  if (batched) why = "batched operands";
  else if (o.block_size != 32 || As->dtype != MX_E8M0) why = "only E8M0 scales with block 32 are MFMA-native";
  else if (!pair_supported_by_mfma(A->dtype, B->dtype)) why = "element format pair not instantiated";
  else if (K == 0) why = "K is zero";
  else if ((why = mfma_operand_issue(A->ptr, M, a_ld, A->stride[1], A->dtype, A->packed_dim == 1))) {}
  else if ((why = mfma_operand_issue(B->ptr, N, b_ld, B->stride[0], B->dtype, B->packed_dim == 0))) {}
  else if (C->stride[1] != 1) why = "C is not row-major";
  else if (M >= (1 << 30) || N >= (1 << 30) || K >= (1 << 30)) why = "extent too large";

  int kernel = o.kernel;
  if (kernel == MX_KERNEL_AUTO) {
    if (why) kernel = MX_KERNEL_GENERIC;
    else if (M <= kDecodeAutoM && o.split_k <= 1 && A->dtype != MX_E2M1 && B->dtype == MX_E2M1 &&
             o.a_scale_layout == MX_SCALE_2D &&
             o.b_scale_layout == MX_SCALE_2D && Bs->stride[0] == 1 && As->stride[1] == 1 && K % 512 == 0 &&
             N % 16 == 0 && Bs->stride[1] % 16 == 0 && ((uintptr_t)Bs->ptr) % 16 == 0 &&
             N * b_ld < ((int64_t)1 << 31) && As->stride[0] % 16 == 0 && ((uintptr_t)As->ptr) % 16 == 0)
      kernel = MX_KERNEL_DECODE;
    else if (big_tile_problem(M, N)) kernel = big_tile_kernel();
    else kernel = MX_KERNEL_MFMA_128x128;
  } else if (kernel != MX_KERNEL_GENERIC && why) {
    return set_error(MX_ERR_LAYOUT, "requested kernel %d cannot run this problem: %s", kernel, why);
  }

  if (o.split_k > 1 && kernel != MX_KERNEL_MFMA_128x128 && kernel != MX_KERNEL_MFMA_256x256 &&
      kernel != MX_KERNEL_MFMA_256x256_W4)
    return set_error(MX_ERR_LAYOUT, "split_k = %d is only available on the one-tile MFMA kernels (kernel %d chosen)",
                     o.split_k, kernel);
  if (plan && kernel != MX_KERNEL_MFMA_128x128) return kPlanNotSimple;
  if (kernel == MX_KERNEL_GENERIC) {
    if (is_native(o.a_scale_layout) || is_native(o.b_scale_layout))
      return set_error(MX_ERR_LAYOUT, "the generic kernel cannot read native-layout scales");
    if (As->dtype == MX_E4M3 && !(A->dtype == MX_E2M1 && o.block_size == 16))
      return set_error(MX_ERR_DTYPE, "E4M3 scales are only defined for FP4 operands with block size 16");
    if (o.block_size == 16 && (A->dtype != MX_E2M1 || B->dtype != MX_E2M1))
      return set_error(MX_ERR_DTYPE, "block size 16 is only defined for FP4 operands");
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF || batch > 0x7FFFFFFF)
      return set_error(MX_ERR_SHAPE, "extents of 2^31 or more are not supported");
    if ((o.a_scale_layout == MX_SCALE_SWIZZLE_32_4_4 || o.b_scale_layout == MX_SCALE_SWIZZLE_32_4_4) && batched)
      return set_error(MX_ERR_LAYOUT, "swizzled scale tensors have no batch dimension");
    if (o.a_scale_layout == MX_SCALE_SWIZZLE_32_4_4)
      if (int rc = check_swizzled_scale(As, "A_scale", M, KB)) return rc;
    if (o.b_scale_layout == MX_SCALE_SWIZZLE_32_4_4)
      if (int rc = check_swizzled_scale(Bs, "B_scale", N, KB)) return rc;
    GenericArgs g = {};
    g.A = (const uint8_t*)A->ptr; g.As = (const uint8_t*)As->ptr;
    g.B = (const uint8_t*)B->ptr; g.Bs = (const uint8_t*)Bs->ptr; g.C = C->ptr;
    g.batch = (int32_t)batch; g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)K; g.block = o.block_size;
    g.a_fmt = A->dtype; g.b_fmt = B->dtype; g.scale_fmt = As->dtype; g.c_dtype = C->dtype;
    g.accumulate = o.accumulate;
    g.a_packed_k = A->packed_dim == and_ - 1; g.b_packed_k = B->packed_dim == bnd - 2;
    g.a_sb = (and_ == 3 && batchA > 1) ? A->stride[0] : 0;
    g.a_sm = A->stride[and_ - 2]; g.a_sk = A->stride[and_ - 1];
    g.b_sb = (bnd == 3 && batchB > 1) ? B->stride[0] : 0;
    g.b_sk = B->stride[bnd - 2]; g.b_sn = B->stride[bnd - 1];
    g.as_layout = o.a_scale_layout; g.bs_layout = o.b_scale_layout;
    if (o.a_scale_layout == MX_SCALE_2D) {
      const int nd = As->ndim;
      g.as_sb = (nd == 3 && batchA > 1) ? As->stride[0] : 0;
      g.as_sm = As->stride[nd - 2]; g.as_sk = As->stride[nd - 1];
    }
    if (o.b_scale_layout == MX_SCALE_2D) {
      const int nd = Bs->ndim;
      g.bs_sb = (nd == 3 && batchB > 1) ? Bs->stride[0] : 0;
      g.bs_sk = Bs->stride[nd - 2]; g.bs_sn = Bs->stride[nd - 1];
    }
    g.c_sb = cnd == 3 ? C->stride[0] : 0; g.c_sm = C->stride[cnd - 2]; g.c_sn = C->stride[cnd - 1];
    return launch_gemm_generic(g, (hipStream_t)stream);
  }

  if (kernel == MX_KERNEL_DECODE) {
    if (M > kDecodeMaxM)
      return set_error(MX_ERR_SHAPE, "the decode kernel handles M <= %lld (got %lld)", (long long)kDecodeMaxM, (long long)M);
    if (o.a_scale_layout != MX_SCALE_2D || o.b_scale_layout != MX_SCALE_2D || Bs->stride[0] != 1 ||
        As->stride[1] != 1)
      return set_error(MX_ERR_LAYOUT, "the decode kernel reads K-contiguous 2-D scales in place");
    if (A->dtype == MX_E2M1 || B->dtype != MX_E2M1)
      return set_error(MX_ERR_DTYPE, "the decode kernel takes 8-bit activations and FP4 weights");
    if (K % 512 != 0 || N % 16 != 0)
      return set_error(MX_ERR_SHAPE, "the decode kernel needs K %% 512 == 0 and N %% 16 == 0");
    DecodeArgs d = {};
    d.X = (const uint8_t*)A->ptr; d.Xs = (const uint8_t*)As->ptr;
    d.W = (const uint8_t*)B->ptr; d.Ws = (const uint8_t*)Bs->ptr; d.C = C->ptr;
    d.M = (int32_t)M; d.N = (int32_t)N; d.K = (int32_t)K;
    d.ldx = a_ld; d.ldxs = As->stride[0]; d.ldw = b_ld; d.ldws = Bs->stride[1]; d.ldc = C->stride[0];
    d.x_fmt = A->dtype; d.w_fmt = B->dtype; d.c_dtype = C->dtype; d.accumulate = o.accumulate;
    const int c_bytes = C->dtype == MX_BF16 ? 2 : 4;
    // slabs of 32 rows of X (and of C, or of the chunk buffer)
    auto launch_slabs = [&](const DecodeArgs& full, int out_bytes) {
      for (int64_t m0 = 0; m0 < M; m0 += 32) {
        DecodeArgs s = full;
        s.X = full.X + m0 * full.ldx; s.Xs = full.Xs + m0 * full.ldxs;
        s.C = (uint8_t*)full.C + m0 * full.ldc * out_bytes;
        s.M = (int32_t)(M - m0 < 32 ? M - m0 : 32);
        if (int rc = launch_gemm_decode(s, (hipStream_t)stream)) return rc;
      }
      return (int)MX_OK;
    };
    if (K <= kDecodeChunk) return launch_slabs(d, c_bytes);
    // a longer K (the down-projection of an MoE layer, K = 14336 / 28672): chunks of kDecodeChunk elements, each
    // streaming its part of the weights once, summed in fp32 in the workspace in chunk order
    const int64_t need = decode_partial_bytes(M, N, K, o);
    if (!workspace || workspace_bytes < need)
      return set_error(MX_ERR_WORKSPACE, "workspace of %lld bytes required, %lld given", (long long)need,
                       (long long)workspace_bytes);
    if (((uintptr_t)workspace) % 256 != 0) return set_error(MX_ERR_WORKSPACE, "workspace must be 256-byte aligned");
    for (int64_t k0 = 0; k0 < K; k0 += kDecodeChunk) {
      DecodeArgs c = d;
      c.X = d.X + k0; c.Xs = d.Xs + k0 / 32;          // 8-bit activations: one byte per element
      c.W = d.W + k0 / 2; c.Ws = d.Ws + k0 / 32;      // FP4 weights: two elements per byte
      c.K = (int32_t)(K - k0 < kDecodeChunk ? K - k0 : kDecodeChunk);
      c.C = workspace; c.ldc = N; c.c_dtype = MX_F32; c.accumulate = k0 > 0;
      if (int rc = launch_slabs(c, 4)) return rc;
    }
    return launch_splitk_reduce((const float*)workspace, 1, M, N, C->ptr, C->stride[0], C->dtype, o.accumulate,
                                (hipStream_t)stream);
  }

  // ---- MFMA path: bring the scales into the native layout if they are not ----------------------------
  uint8_t* ws = (uint8_t*)workspace;
  int64_t need = mx_gemm_workspace_bytes(M, N, K, &o);
  if (need > 0 && (!ws || workspace_bytes < need))
    return set_error(MX_ERR_WORKSPACE, "workspace of %lld bytes required, %lld given", (long long)need,
                     (long long)workspace_bytes);
  if (need > 0 && ((uintptr_t)ws) % 256 != 0)
    return set_error(MX_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  const uint32_t* as_native = (const uint32_t*)As->ptr;
  const uint32_t* bs_native = (const uint32_t*)Bs->ptr;
  PackArgs pa, pb;
  int S = 1;
  if (kernel == MX_KERNEL_MFMA_128x128 || kernel == MX_KERNEL_MFMA_256x256 || kernel == MX_KERNEL_MFMA_256x256_W4) {
    S = plan_k_splits(M, N, K, o);
    if (S < 0)
      return set_error(MX_ERR_SHAPE, "split_k = %d needs K (%lld) to be a multiple of %d", o.split_k, (long long)K,
                       512 * o.split_k);
  }
  if (S > 1 && plan) return kPlanNotSimple;
  if (S > 1) {
    // ---- split-K: the slices are a batch for the scale re-layout and a second grid dimension for the GEMM
    const int64_t Ks = K / S, kbs = Ks / 32;
    if (int rc = make_pack_args(As, MX_SCALE_2D, M, K, ws, kPackA, pa)) return rc;
    pa.K = Ks; pa.batch = S; pa.s_batch = kbs * pa.s_kb;
    const uint32_t* as_p = (const uint32_t*)ws;
    ws += S * mx_packed_scale_bytes(M, Ks);
    mx_tensor t = *Bs;   // [K/32, N] -> view as [N, K/32]
    t.shape[0] = Bs->shape[1]; t.shape[1] = Bs->shape[0];
    t.stride[0] = Bs->stride[1]; t.stride[1] = Bs->stride[0];
    if (int rc = make_pack_args(&t, MX_SCALE_2D, N, K, ws, kPackB, pb)) return rc;
    pb.K = Ks; pb.batch = S; pb.s_batch = kbs * pb.s_kb;
    const uint32_t* bs_p = (const uint32_t*)ws;
    ws += S * mx_packed_scale_bytes(N, Ks);
    float* partial = (float*)ws;
    if (int rc = launch_pack_scales_pair(&pa, &pb, (hipStream_t)stream)) return rc;
    GemmArgs g = {};
    g.A = (const uint8_t*)A->ptr; g.B = (const uint8_t*)B->ptr; g.As = as_p; g.Bs = bs_p; g.C = partial;
    g.lda = a_ld; g.ldb = b_ld; g.ldc = N;
    g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)Ks;
    g.a_fmt = A->dtype; g.b_fmt = B->dtype; g.c_dtype = MX_F32; g.accumulate = 0;
    g.a_rows = M;
    g.replicas = 1;
    g.k_splits = S;
    g.as_split_stride = mx_packed_scale_bytes(M, Ks) / 4;
    g.bs_split_stride = mx_packed_scale_bytes(N, Ks) / 4;
    g.c_split_stride = M * N;
    if (int rc = launch_gemm_mfma(g, kernel, (hipStream_t)stream)) return rc;
    return launch_splitk_reduce(partial, S, M, N, C->ptr, C->stride[0], C->dtype, o.accumulate, (hipStream_t)stream);
  }
  // (the decode and general kernels returned above: from here on `kernel` is one that reads a native layout)
  const int native = native_layout_of(kernel);
  const bool pack_a = !is_native(o.a_scale_layout), pack_b = !is_native(o.b_scale_layout);
  if ((!pack_a && o.a_scale_layout != native) || (!pack_b && o.b_scale_layout != native))
    return set_error(MX_ERR_LAYOUT, "kernel %d reads native-layout scales of kind %d (MX_SCALE_NATIVE for the "
                     "16x16x128-instruction kernels, MX_SCALE_NATIVE32 for pingpong32 / w4p); pass the matching "
                     "layout or the plain 2-D scales", kernel, native);
  const bool t32 = native == MX_SCALE_NATIVE32;
  if (pack_a) {
    if (int rc = make_pack_args(As, o.a_scale_layout, M, K, ws, t32 ? kPackTile32 : kPackA, pa)) return rc;
    as_native = (const uint32_t*)ws;
    ws += mx_packed_scale_bytes(M, K);
  }
  if (pack_b) {
    mx_tensor t = *Bs;
    if (o.b_scale_layout == MX_SCALE_2D) {  // [K/32, N] -> view as [N, K/32]
      t.shape[0] = Bs->shape[1]; t.shape[1] = Bs->shape[0];
      t.stride[0] = Bs->stride[1]; t.stride[1] = Bs->stride[0];
    }
    if (int rc = make_pack_args(&t, o.b_scale_layout, N, K, ws, t32 ? kPackTile32 : kPackB, pb)) return rc;
    bs_native = (const uint32_t*)ws;
  }
  if (((uintptr_t)as_native) % 16 != 0 || ((uintptr_t)bs_native) % 16 != 0)
    return set_error(MX_ERR_LAYOUT, "native scale buffers must be 16-byte aligned");
  if (!plan && (pack_a || pack_b))   // one launch for both operands
    if (int rc = launch_pack_scales_pair(pack_a ? &pa : nullptr, pack_b ? &pb : nullptr, (hipStream_t)stream)) return rc;

  GemmArgs g = {};
  g.A = (const uint8_t*)A->ptr; g.B = (const uint8_t*)B->ptr; g.As = as_native; g.Bs = bs_native; g.C = C->ptr;
  g.lda = a_ld; g.ldb = b_ld; g.ldc = C->stride[0];
  g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)K;
  g.a_fmt = A->dtype; g.b_fmt = B->dtype; g.c_dtype = C->dtype; g.accumulate = o.accumulate;
  g.a_rows = M;
  g.replicas = 1;
  if (plan) {
    if ((pack_a && o.a_scale_layout != MX_SCALE_2D) || (pack_b && o.b_scale_layout != MX_SCALE_2D)) return kPlanNotSimple;
    plan->g = g;
    plan->pack_a = pack_a; plan->pack_b = pack_b;
    if (pack_a) plan->pa = pa;
    if (pack_b) plan->pb = pb;
    return MX_OK;
  }
  return launch_gemm_mfma(g, kernel, (hipStream_t)stream);
}
}  // namespace

namespace {
// logical (M, N, K) of a problem from its operand descriptors (FP4 operands count elements, not bytes)
void problem_dims(const mx_tensor& A, const mx_tensor& B, int64_t& M, int64_t& N, int64_t& K) {
  const int an = A.ndim, bn = B.ndim;
  M = an >= 2 ? A.shape[an - 2] : 0;
  K = an >= 2 ? A.shape[an - 1] : 0;
  N = bn >= 2 ? B.shape[bn - 1] : 0;
}
}  // namespace

int64_t mx_static_scratch_bytes(void) { return MX_STATIC_SCRATCH_BYTES; }

int mx_gemm_static(const mx_tensor* A, const mx_tensor* As, const mx_tensor* B, const mx_tensor* Bs, mx_tensor* C,
                   const mx_gemm_opts* opts, void* stream) {
  if (!A || !B) return set_error(MX_ERR_INVALID, "mx_gemm_static: null descriptor");
  if (A->ndim < 2 || A->ndim > 3 || B->ndim < 2 || B->ndim > 3)
    return set_error(MX_ERR_SHAPE, "mx_gemm_static: A and B must have 2 or 3 dimensions");
  int64_t M, N, K;
  problem_dims(*A, *B, M, N, K);
  const int64_t need = mx_gemm_workspace_bytes(M, N, K, opts);
  if (need > MX_STATIC_SCRATCH_BYTES)
    return set_error(MX_ERR_WORKSPACE, "mx_gemm_static: this problem needs %lld bytes of scratch, the static buffer "
                     "holds %lld; use mx_gemm with a caller-owned workspace", (long long)need,
                     (long long)MX_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  return mx_gemm(A, As, B, Bs, C, opts, ws, MX_STATIC_SCRATCH_BYTES, stream);
}

int64_t mx_gemm_list_workspace_bytes(int32_t count, const mx_tensor* A, const mx_tensor* B,
                                     const mx_gemm_opts* opts) {
  if (count <= 0 || !A || !B) return 0;
  int64_t need = 0;   // every problem has its own slice: the problems of a list run side by side
  for (int32_t i = 0; i < count; ++i) {
    int64_t M, N, K;
    problem_dims(A[i], B[i], M, N, K);
    need += round256(mx_gemm_workspace_bytes(M, N, K, opts));
  }
  return need;
}

int mx_gemm_list(int32_t count, const mx_tensor* A, const mx_tensor* As, const mx_tensor* B, const mx_tensor* Bs,
                 mx_tensor* C, const mx_gemm_opts* opts, void* workspace, int64_t workspace_bytes, void* stream) {
  if (count < 0) return set_error(MX_ERR_INVALID, "mx_gemm_list: negative count");
  if (count == 0) return MX_OK;
  if (!A || !As || !B || !Bs || !C) return set_error(MX_ERR_INVALID, "mx_gemm_list: null descriptor array");
  const int64_t need = mx_gemm_list_workspace_bytes(count, A, B, opts);
  if (need > 0 && (!workspace || workspace_bytes < need))
    return set_error(MX_ERR_WORKSPACE, "workspace of %lld bytes required, %lld given", (long long)need,
                     (long long)workspace_bytes);
  if (need > 0 && ((uintptr_t)workspace) % 256 != 0) return set_error(MX_ERR_WORKSPACE, "workspace must be 256-byte aligned");

  // Pass 1: validate everything and sort the problems: those that would run on the 128 x 128 one-tile kernel are
  // collected (no launch), the others are remembered for a call of their own.  Nothing is enqueued if any problem
  // is invalid.
  struct Item { int32_t index; int64_t ws_off, ws_bytes; bool simple; GemmPlan plan; };
  std::vector<Item> items;
  items.reserve(count);
  int64_t off = 0;
  for (int32_t i = 0; i < count; ++i) {
    int64_t M, N, K;
    problem_dims(A[i], B[i], M, N, K);
    const int64_t b = round256(mx_gemm_workspace_bytes(M, N, K, opts));
    Item it = {};
    it.index = i; it.ws_off = off; it.ws_bytes = b;
    off += b;
    if (A[i].ndim == 2 && B[i].ndim == 2 && (M == 0 || N == 0)) continue;   // empty problem
    const int rc = gemm_impl(&A[i], &As[i], &B[i], &Bs[i], &C[i], opts, (uint8_t*)workspace + it.ws_off, it.ws_bytes,
                             stream, &it.plan);
    if (rc < 0) {
      char inner[400];
      snprintf(inner, sizeof inner, "%s", mx_last_error());
      return set_error(rc, "problem %d of the list: %s", (int)i, inner);
    }
    it.simple = rc == MX_OK;
    items.push_back(it);
  }
  // Pass 2: one scale re-layout launch per 64 scale tensors, one persistent GEMM launch per 32 problems of one
  // element-format pair and output type
  std::vector<PackArgs> packs;
  for (const Item& it : items) {
    if (!it.simple) continue;
    if (it.plan.pack_a) packs.push_back(it.plan.pa);
    if (it.plan.pack_b) packs.push_back(it.plan.pb);
  }
  if (!packs.empty())
    if (int rc = launch_pack_scales_list(packs.data(), (int)packs.size(), (hipStream_t)stream)) return rc;
  std::vector<char> done(items.size(), 0);
  for (size_t i = 0; i < items.size(); ++i) {
    if (!items[i].simple || done[i]) continue;
    std::vector<GemmArgs> group;
    const GemmArgs& g0 = items[i].plan.g;
    for (size_t j = i; j < items.size(); ++j) {
      const GemmArgs& g = items[j].plan.g;
      if (items[j].simple && !done[j] && g.a_fmt == g0.a_fmt && g.b_fmt == g0.b_fmt && g.c_dtype == g0.c_dtype) {
        group.push_back(g);
        done[j] = 1;
      }
    }
    if (int rc = launch_gemm_mfma_list(group.data(), (int)group.size(), (hipStream_t)stream)) return rc;
  }
  // Pass 3: the rest (large problems for the persistent 256 x 256 kernel, skinny ones for the decode kernel,
  // split-K, batched operands, layouts only the general kernel reads), one call each
  for (const Item& it : items) {
    if (it.simple) continue;
    const int32_t i = it.index;
    const int rc = mx_gemm(&A[i], &As[i], &B[i], &Bs[i], &C[i], opts, (uint8_t*)workspace + it.ws_off, it.ws_bytes, stream);
    if (rc != MX_OK) {
      char inner[400];
      snprintf(inner, sizeof inner, "%s", mx_last_error());
      return set_error(rc, "problem %d of the list: %s", (int)i, inner);
    }
  }
  return MX_OK;
}

int mx_bench_gemm(int32_t nsets, const mx_tensor* A, const mx_tensor* As, const mx_tensor* B, const mx_tensor* Bs,
                  mx_tensor* C, const mx_gemm_opts* opts, void* workspace, int64_t workspace_bytes, int32_t warmup,
                  int32_t iters, float* times_ms, void* stream) {
  if (nsets <= 0 || !A || !As || !B || !Bs || !C) return set_error(MX_ERR_INVALID, "mx_bench_gemm: no operand sets");
  if (warmup < 0 || iters <= 0 || iters > 65536 || !times_ms)
    return set_error(MX_ERR_INVALID, "mx_bench_gemm: iters must be in 1..65536 and times_ms non-null");
  hipStream_t st = (hipStream_t)stream;
  for (int i = 0; i < warmup; ++i) {
    const int s = i % nsets;
    if (int rc = mx_gemm(&A[s], &As[s], &B[s], &Bs[s], &C[s], opts, workspace, workspace_bytes, stream)) return rc;
  }
  hipEvent_t* ev = (hipEvent_t*)calloc((size_t)2 * iters, sizeof(hipEvent_t));
  if (!ev) return set_error(MX_ERR_INVALID, "mx_bench_gemm: out of host memory");
  int rc = MX_OK, made = 0;
  for (; made < 2 * iters; ++made)
    if (hipEventCreate(&ev[made]) != hipSuccess) { rc = set_error(MX_ERR_DEVICE, "mx_bench_gemm: hipEventCreate failed"); break; }
  for (int i = 0; rc == MX_OK && i < iters; ++i) {
    const int s = (warmup + i) % nsets;
    if (hipEventRecord(ev[2 * i], st) != hipSuccess) { rc = set_error(MX_ERR_DEVICE, "mx_bench_gemm: hipEventRecord failed"); break; }
    rc = mx_gemm(&A[s], &As[s], &B[s], &Bs[s], &C[s], opts, workspace, workspace_bytes, stream);
    if (rc == MX_OK && hipEventRecord(ev[2 * i + 1], st) != hipSuccess)
      rc = set_error(MX_ERR_DEVICE, "mx_bench_gemm: hipEventRecord failed");
  }
  // the stream is drained on every path, so that no event is destroyed while still pending
  const hipError_t es = hipStreamSynchronize(st);
  if (rc == MX_OK && es != hipSuccess) rc = set_error(MX_ERR_DEVICE, "mx_bench_gemm: %s", hipGetErrorString(es));
  for (int i = 0; rc == MX_OK && i < iters; ++i)
    if (hipEventElapsedTime(&times_ms[i], ev[2 * i], ev[2 * i + 1]) != hipSuccess)
      rc = set_error(MX_ERR_DEVICE, "mx_bench_gemm: hipEventElapsedTime failed");
  for (int i = 0; i < made; ++i) (void)hipEventDestroy(ev[i]);
  free(ev);
  return rc;
}

int mx_gemm_grouped(const mx_tensor* A, const mx_tensor* As, const mx_tensor* W, const mx_tensor* Ws,
                    mx_tensor* C, const float* topk_weights, const int32_t* sorted_token_ids,
                    int64_t num_slots, const int32_t* sorted_expert_ids, int32_t tile_m,
                    int32_t num_token_replicas, int64_t num_valid_ids, const mx_gemm_opts* opts,
                    void* workspace, int64_t workspace_bytes, void* stream) {
  const mx_gemm_opts& o = opts ? *opts : kDefaultOpts;
  if (int rc = check_tensor(A, "A", 2, 2)) return rc;
  if (int rc = check_tensor(As, "A_scale", 2, 2)) return rc;
  if (int rc = check_tensor(W, "W", 3, 3)) return rc;
  if (int rc = check_tensor(Ws, "W_scale", 3, 3)) return rc;
  if (int rc = check_tensor(C, "C", 2, 2)) return rc;
  if (!sorted_token_ids || !sorted_expert_ids) return set_error(MX_ERR_INVALID, "null index arrays");
  if (tile_m <= 0 || num_slots % tile_m != 0)
    return set_error(MX_ERR_SHAPE, "num_slots (%lld) must be a multiple of tile_m (%d)", (long long)num_slots, tile_m);
  if (num_token_replicas <= 0) return set_error(MX_ERR_INVALID, "num_token_replicas must be positive");
  if (!is_elem(A->dtype) || !is_elem(W->dtype)) return set_error(MX_ERR_DTYPE, "A/W must be MX element formats");
  if (As->dtype != MX_E8M0 || Ws->dtype != MX_E8M0) return set_error(MX_ERR_DTYPE, "scales must be MX_E8M0");
  if (C->dtype != MX_F32 && C->dtype != MX_BF16) return set_error(MX_ERR_DTYPE, "C must be MX_F32 or MX_BF16");
  if (o.block_size != 32) return set_error(MX_ERR_INVALID, "grouped GEMM supports block size 32 only");
  const int64_t T = A->shape[0], K = A->shape[1], E = W->shape[0], N = W->shape[1];
  if (W->shape[2] != K)
    return set_error(MX_ERR_SHAPE, "Incompatible matrices: K dimension of A (%lld) must match K dimension of W (%lld)",
                     (long long)K, (long long)W->shape[2]);
  if (K % 32 != 0) return set_error(MX_ERR_SHAPE, "K (%lld) must be a multiple of 32", (long long)K);
  const int64_t KB = K / 32;
  if (As->shape[0] != T || As->shape[1] != KB) return set_error(MX_ERR_SHAPE, "A_scale must be [tokens, K/32]");
  if (!is_native(o.b_scale_layout) && (Ws->shape[0] != E || Ws->shape[1] != N || Ws->shape[2] != KB))
    return set_error(MX_ERR_SHAPE, "W_scale must be [experts, N, K/32]");
  if (C->shape[1] != N || C->shape[0] < num_valid_ids)
    return set_error(MX_ERR_SHAPE, "C must be [>= num_valid_ids, N]");
  if ((num_valid_ids + num_token_replicas - 1) / num_token_replicas > T)
    return set_error(MX_ERR_SHAPE, "num_valid_ids / num_token_replicas exceeds the rows of A");
  if (num_slots == 0 || N == 0) return MX_OK;
  if (E <= 0 || E > 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "W must hold at least one expert");
  if (A->dtype == MX_E2M1 && A->packed_dim != 1) return set_error(MX_ERR_LAYOUT, "A must be packed along K");
  if (W->dtype == MX_E2M1 && W->packed_dim != 2) return set_error(MX_ERR_LAYOUT, "W must be packed along K");

  const char* why = nullptr;
  if (!pair_supported_by_mfma(A->dtype, W->dtype)) why = "element format pair not instantiated";
  else if ((why = mfma_operand_issue(A->ptr, T, A->stride[0], A->stride[1], A->dtype, 1))) {}
  else if ((why = mfma_operand_issue(W->ptr, N, W->stride[1], W->stride[2], W->dtype, 1))) {}
  else if (W->stride[0] % 16 != 0) why = "expert pitch of W is not a multiple of 16 bytes";
  else if (C->stride[1] != 1) why = "C is not row-major";
  else if (tile_m % 128 != 0) why = "tile_m is not a multiple of 128";
  else if (o.a_scale_layout != MX_SCALE_2D) why = "A_scale must be the plain 2-D layout";

  int kernel = o.kernel;
  if (kernel == MX_KERNEL_AUTO) {
    if (why) kernel = MX_KERNEL_GENERIC;
    else kernel = (tile_m % 256 == 0 && N > 128) ? big_tile_kernel() : MX_KERNEL_MFMA_128x128;
  } else if (kernel != MX_KERNEL_GENERIC) {
    if (why) return set_error(MX_ERR_LAYOUT, "requested kernel %d cannot run this problem: %s", kernel, why);
    const int bm = kernel == MX_KERNEL_MFMA_128x128 ? 128 : 256;
    if (kernel == MX_KERNEL_DECODE || tile_m % bm != 0)
      return set_error(MX_ERR_LAYOUT, "kernel %d needs tile_m to be a multiple of its row tile", kernel);
  }

  if (kernel == MX_KERNEL_GENERIC) {
    if (o.a_scale_layout != MX_SCALE_2D || o.b_scale_layout != MX_SCALE_2D)
      return set_error(MX_ERR_LAYOUT, "the generic grouped kernel reads plain 2-D / 3-D scales");
    GenericArgs g = {};
    g.A = (const uint8_t*)A->ptr; g.As = (const uint8_t*)As->ptr;
    g.B = (const uint8_t*)W->ptr; g.Bs = (const uint8_t*)Ws->ptr; g.C = C->ptr;
    g.batch = 1; g.M = (int32_t)T; g.N = (int32_t)N; g.K = (int32_t)K; g.block = 32;
    g.a_fmt = A->dtype; g.b_fmt = W->dtype; g.scale_fmt = MX_E8M0; g.c_dtype = C->dtype; g.accumulate = o.accumulate;
    g.a_packed_k = 1; g.b_packed_k = 1;
    g.a_sm = A->stride[0]; g.a_sk = A->stride[1];
    g.as_sm = As->stride[0]; g.as_sk = As->stride[1];
    g.b_sn = W->stride[1]; g.b_sk = W->stride[2]; g.b_se = W->stride[0];
    g.bs_sn = Ws->stride[1]; g.bs_sk = Ws->stride[2]; g.bs_se = Ws->stride[0];
    g.c_sm = C->stride[0]; g.c_sn = C->stride[1];
    g.sorted_token_ids = sorted_token_ids; g.sorted_expert_ids = sorted_expert_ids; g.topk_weights = topk_weights;
    g.tile_m = tile_m; g.replicas = num_token_replicas; g.num_valid_ids = num_valid_ids; g.num_slots = num_slots;
    g.num_experts = (int32_t)E;
    return launch_gemm_generic(g, (hipStream_t)stream);
  }

  uint8_t* ws = (uint8_t*)workspace;
  const int64_t need = mx_gemm_grouped_workspace_bytes(num_slots, N, K, E, &o);
  if (!ws || workspace_bytes < need)
    return set_error(MX_ERR_WORKSPACE, "workspace of %lld bytes required, %lld given", (long long)need,
                     (long long)workspace_bytes);
  if (((uintptr_t)ws) % 256 != 0) return set_error(MX_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  // A scales: gathered into slot order while re-laying; W scales of all experts ride in the same launch
  const int native = native_layout_of(kernel);
  const bool t32 = native == MX_SCALE_NATIVE32;
  PackArgs pa = {}, pw;
  pa.target = t32 ? kPackTile32 : kPackA;
  pa.src = (const uint8_t*)As->ptr; pa.dst = (uint32_t*)ws;
  pa.rows = num_slots; pa.K = K; pa.s_row = As->stride[0]; pa.s_kb = As->stride[1];
  pa.layout = MX_SCALE_2D; pa.batch = 1;
  pa.gather_ids = sorted_token_ids; pa.replicas = num_token_replicas; pa.num_valid_ids = num_valid_ids;
  const uint32_t* as_native = (const uint32_t*)ws;
  ws += mx_packed_scale_bytes(num_slots, K);
  const uint32_t* bs_native = (const uint32_t*)Ws->ptr;
  const bool pack_w = !is_native(o.b_scale_layout);
  if (!pack_w && o.b_scale_layout != native)
    return set_error(MX_ERR_LAYOUT, "kernel %d reads native-layout scales of kind %d, W_scale has kind %d", kernel,
                     native, o.b_scale_layout);
  if (E * mx_packed_scale_bytes(N, K) >= ((int64_t)1 << 31))
    return set_error(MX_ERR_SHAPE, "the packed scales of all experts must stay below 2 GiB");
  if (pack_w) {
    if (o.b_scale_layout != MX_SCALE_2D) return set_error(MX_ERR_LAYOUT, "W_scale must be [E, N, K/32] or native");
    if (int rc = make_pack_args(Ws, MX_SCALE_2D, N, K, ws, t32 ? kPackTile32 : kPackB, pw)) return rc;
    bs_native = (const uint32_t*)ws;
  }
  if (int rc = launch_pack_scales_pair(&pa, pack_w ? &pw : nullptr, (hipStream_t)stream)) return rc;
  GemmArgs g = {};
  g.A = (const uint8_t*)A->ptr; g.B = (const uint8_t*)W->ptr; g.As = as_native; g.Bs = bs_native; g.C = C->ptr;
  g.lda = A->stride[0]; g.ldb = W->stride[1]; g.ldc = C->stride[0];
  g.M = (int32_t)num_slots; g.N = (int32_t)N; g.K = (int32_t)K;
  g.a_fmt = A->dtype; g.b_fmt = W->dtype; g.c_dtype = C->dtype; g.accumulate = o.accumulate;
  g.sorted_token_ids = sorted_token_ids; g.sorted_expert_ids = sorted_expert_ids; g.topk_weights = topk_weights;
  g.tile_m = tile_m; g.replicas = num_token_replicas; g.num_valid_ids = num_valid_ids;
  g.num_experts = (int32_t)E;
  g.b_expert_stride = W->stride[0];
  g.bs_expert_stride = mx_packed_scale_bytes(N, K) / 4;
  g.a_rows = T;
  return launch_gemm_mfma(g, kernel, (hipStream_t)stream);
}

int64_t mx_moe_align_max_slots(int64_t num_ids, int32_t num_experts, int32_t tile_m) {
  if (num_ids < 0 || num_experts <= 0 || tile_m <= 0) return 0;
  const int64_t nonempty = num_experts < num_ids ? num_experts : num_ids;
  return (num_ids + nonempty * (tile_m - 1)) / tile_m * tile_m;
}

int64_t mx_moe_align_workspace_bytes(int64_t num_ids, int32_t num_experts) {
  if (num_ids <= 0 || num_experts <= 0) return 0;
  return round256(moe_align_workspace_bytes(num_ids, num_experts));
}

int mx_moe_align(const int32_t* topk_ids, int64_t num_ids, int32_t num_experts, int32_t tile_m,
                 int32_t* sorted_token_ids, int32_t* sorted_expert_ids, int32_t* num_slots_out, void* workspace,
                 int64_t workspace_bytes, void* stream) {
  if (num_ids < 0 || num_experts <= 0 || tile_m <= 0) return set_error(MX_ERR_INVALID, "moe_align: bad sizes");
  if (num_ids >= 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "moe_align: too many ids");
  const int64_t max_slots = mx_moe_align_max_slots(num_ids, num_experts, tile_m);
  if (max_slots == 0) {
    return MX_OK;
  }
  if (max_slots >= 0x7FFFFFFF) return set_error(MX_ERR_SHAPE, "moe_align: too many slots");
  if (!topk_ids || !sorted_token_ids || !sorted_expert_ids) return set_error(MX_ERR_INVALID, "moe_align: null pointer");
  const int64_t need = moe_align_workspace_bytes(num_ids, num_experts);
  if (need > 0 && (!workspace || workspace_bytes < need))
    return set_error(MX_ERR_WORKSPACE, "moe_align: workspace of %lld bytes required, %lld given", (long long)need,
                     (long long)workspace_bytes);
  if (need > 0 && ((uintptr_t)workspace) % 4 != 0) return set_error(MX_ERR_WORKSPACE, "moe_align: workspace must be 4-byte aligned");
  return launch_moe_align(topk_ids, num_ids, num_experts, tile_m, sorted_token_ids, sorted_expert_ids,
                          num_slots_out, max_slots, (int32_t*)workspace, (hipStream_t)stream);
}

namespace {
// shared by mx_quantize and mx_silu_mul_quantize; K = quantised row length, `up` null for the plain form
int quantize_common(const mx_tensor* x, const void* up, int64_t K, mx_tensor* xq, mx_tensor* scale,
                    int32_t scale_mode, void* stream) {
  if (int rc = check_tensor(xq, "xq", 2, 2)) return rc;
  if (int rc = check_tensor(scale, "scale", 2, 2)) return rc;
  if (x->dtype != MX_F32 && x->dtype != MX_BF16 && x->dtype != MX_F16)
    return set_error(MX_ERR_DTYPE, "x must be MX_F32, MX_BF16 or MX_F16");
  if (!is_elem(xq->dtype)) return set_error(MX_ERR_DTYPE, "xq must be an MX element format");
  if (scale->dtype != MX_E8M0) return set_error(MX_ERR_DTYPE, "scale must be MX_E8M0");
  if (scale_mode != 0 && scale_mode != 1) return set_error(MX_ERR_INVALID, "scale_mode must be 0 (ceil) or 1 (floor)");
  const int64_t rows = x->shape[0];
  if (K < 32)
    return set_error(MX_ERR_SHAPE,
                     "The requested block size 32 is larger than the inner most dimension of the input tensor %lld",
                     (long long)K);
  const int64_t Kpad = (K + 31) / 32 * 32;
  if (xq->shape[0] != rows || xq->shape[1] != Kpad || scale->shape[0] != rows || scale->shape[1] != Kpad / 32)
    return set_error(MX_ERR_SHAPE, "xq must be [rows, %lld] and scale [rows, %lld]", (long long)Kpad,
                     (long long)(Kpad / 32));
  if (x->stride[1] != 1 || xq->stride[1] != 1 || scale->stride[1] != 1)
    return set_error(MX_ERR_LAYOUT, "x, xq and scale must be contiguous along the last axis");
  if (xq->dtype == MX_E2M1 && xq->packed_dim != 1) return set_error(MX_ERR_LAYOUT, "xq must be packed along K");
  QuantArgs q = {};
  q.x = x->ptr; q.xq = (uint8_t*)xq->ptr; q.scale = (uint8_t*)scale->ptr;
  q.rows = rows; q.K = K; q.Kpad = Kpad;
  q.x_ld = x->stride[0]; q.xq_ld = xq->stride[0]; q.sc_ld = scale->stride[0];
  q.x_dtype = x->dtype; q.fmt = xq->dtype; q.scale_mode = scale_mode;
  q.up = up;
  return launch_quantize(q, (hipStream_t)stream);
}
}  // namespace

int mx_quantize(const mx_tensor* x, mx_tensor* xq, mx_tensor* scale, int32_t scale_mode, void* stream) {
  if (int rc = check_tensor(x, "x", 2, 2)) return rc;
  return quantize_common(x, nullptr, x->shape[1], xq, scale, scale_mode, stream);
}

int mx_silu_mul_quantize(const mx_tensor* gate_up, mx_tensor* xq, mx_tensor* scale, int32_t scale_mode,
                         void* stream) {
  if (int rc = check_tensor(gate_up, "gate_up", 2, 2)) return rc;
  if (gate_up->shape[1] % 2 != 0)
    return set_error(MX_ERR_SHAPE, "gate_up must have an even number of columns (gate | up), got %lld",
                     (long long)gate_up->shape[1]);
  const int64_t F = gate_up->shape[1] / 2;
  const int esz = gate_up->dtype == MX_F32 ? 4 : 2;
  const void* up = (const uint8_t*)gate_up->ptr + F * esz;
  return quantize_common(gate_up, up, F, xq, scale, scale_mode, stream);
}

}  // extern "C"
