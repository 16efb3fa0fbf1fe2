// gfx950 (MI355X, CDNA4) kernels for the fused fp8 LM-head + tanh-softcap + cross-entropy
// loss head, and the C ABI declared in include/slowrun_ce.h.
//
// Replaces, in the reference: the quantise / _scaled_mm / ce_fwd_bwd / transpose_copy chain of
// FusedSoftcappedCrossEntropy (tiny/cuda_kernels.py:336-414, kernel at :125-302).
//
// Data flow
//   forward : X, W --quantise--> X_q [Np][dp], W_q^T [Vp][dp], W_q [dq][Vp]   (OCP e4m3, zero padded)
//             fwd_kernel: 256x256 logit tiles on v_mfma_f32_32x32x64_f8f6f4; the epilogue keeps per-row
//             sum exp(z - cap), the target logits and (on request) max/argmax of u; the logits never leave
//             the chip.  With dlogits_from_forward it also leaves D = (1 - t^2) exp(z - cap) as e4m3 bytes
//             with one power-of-two exponent per 32 rows x 128 columns (G, tile by tile), the targets'
//             entries zero.  Partials per (row, V-split) -> combine.
//   backward: the dlogits as forward left them, or formed again panel by panel from recomputed logit tiles
//             (bwd_recompute_kernel, same format); dX = rho_row * D W_q^T and dW = (rho X_q)^T D run on the
//             same MFMA main loop with the exponents applied inside v_mfma_scale_f32_32x32x64_f8f6f4.  The
//             one-hot part of dlogits never goes through fp8: it is applied in fp32 in the dX epilogue
//             (gather of W_q^T rows) and in the dW finalisation (rows grouped by target).
#include "sce_common.h"
#include "sce_mainloop.h"
#include "../../include/slowrun_ce.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <atomic>
#include <mutex>
#include <type_traits>
#include <vector>

#include "sce_device_util.h"
#include "sce_quantize.h"
#include "sce_dlogits.h"
#include "sce_forward.h"
#include "sce_backward.h"
#include "sce_bench_kernels.h"

// ==========================================================================================
// host side: C ABI
// ==========================================================================================
namespace sce {
int sort_pairs(void* tmp, size_t* tmp_bytes, const int32_t* kin, int32_t* kout, const int32_t* vin, int32_t* vout,
               size_t n, int end_bit, hipStream_t stream);   // sce_sort.hip
}

using namespace sce;

static thread_local char g_err[512] = "";

static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define HIP_TRY(expr)                                                                              \
  do {                                                                                             \
    hipError_t e_ = (expr);                                                                        \
    if (e_ != hipSuccess) return fail(SCE_EHIP, "%s failed: %s", #expr, hipGetErrorString(e_));    \
  } while (0)

struct DeviceGuard {
  int prev = -1;
  bool ok = true;
  explicit DeviceGuard(int dev) {
    if (hipGetDevice(&prev) != hipSuccess) { ok = false; return; }
    if (prev != dev && hipSetDevice(dev) != hipSuccess) ok = false;
  }
  ~DeviceGuard() { if (prev >= 0) (void)hipSetDevice(prev); }
};

// Scratch of sce_forward_noalloc: the V-split partial records of the forward kernel (what sce_forward takes from the
// caller's workspace).  Every GPU the library runs on holds its own copy until the process ends; in host code the
// array's name is only a handle, the address on a device comes from hipGetSymbolAddress (g_scratch, below).
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

static std::mutex g_mu;
static std::atomic<int64_t> g_gather_limit{(int64_t)1 << 32};   // see sce_test_set_gather_limit
static int g_arch_ok[64];   // 0 unknown, 1 gfx950, -1 other
static void* g_scratch[64]; // device address of `scratch` on each device, filled with g_arch_ok
static int g_cus[64];       // compute units, filled with g_arch_ok
static inline int device_cus_or_default(int dev) { return (dev >= 0 && dev < 64 && g_cus[dev] > 0) ? g_cus[dev] : 256; }

// Optional per-kernel timing with HIP events on the caller's stream (off by default).
struct TimingState {
  bool on = false;
  std::vector<hipEvent_t> pool;                       // unused events
  std::vector<hipEvent_t> begin[SCE_K_COUNT], end[SCE_K_COUNT];
  double ms[SCE_K_COUNT] = {0};
  int64_t launches[SCE_K_COUNT] = {0};
};
static TimingState g_timing;
static std::mutex g_timing_mu;

static hipEvent_t timing_event() {
  if (!g_timing.pool.empty()) { hipEvent_t e = g_timing.pool.back(); g_timing.pool.pop_back(); return e; }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}
struct KernelTimer {   // records an event pair around the launches made while it lives
  int kind; hipStream_t st; bool active;
  KernelTimer(int k, hipStream_t s) : kind(k), st(s), active(false) {
    std::lock_guard<std::mutex> lk(g_timing_mu);
    if (!g_timing.on) return;
    hipEvent_t e = timing_event();
    if (!e) return;
    (void)hipEventRecord(e, st);
    g_timing.begin[kind].push_back(e);
    active = true;
  }
  ~KernelTimer() {
    if (!active) return;
    std::lock_guard<std::mutex> lk(g_timing_mu);
    hipEvent_t e = timing_event();
    if (!e) { g_timing.pool.push_back(g_timing.begin[kind].back()); g_timing.begin[kind].pop_back(); return; }
    (void)hipEventRecord(e, st);
    g_timing.end[kind].push_back(e);
  }
};

// First use of a device: its architecture, and the kernels' LDS limits, set with that device current.  A device
// counts as known only once every step has succeeded, so a failure here is tried again on the next call.
static int check_device(int dev) {
  if (dev < 0 || dev >= 64) return fail(SCE_EINVAL, "device %d out of range", dev);
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_arch_ok[dev] == 0) {
    DeviceGuard guard(dev);
    if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", dev);
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
      g_arch_ok[dev] = -1;
    } else {
      // the MFMA kernels hold two 64 KB K-slots in LDS, and more behind them
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<true, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_sample_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_SAMPLE));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_sample_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_SAMPLE));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_sample_kernel<true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_SAMPLE));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<false, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_recompute_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_RECOMPUTE));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<float, false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<bf16_t, false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<float, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<bf16_t, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dw_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dw_tail_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dw_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      void* sp = nullptr;
      HIP_TRY(hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)));       // this device's copy of the array
      g_scratch[dev] = sp;
      g_cus[dev] = prop.multiProcessorCount;
      g_arch_ok[dev] = 1;
    }
  }
  if (g_arch_ok[dev] != 1) return fail(SCE_EARCH, "device %d is not gfx950", dev);
  return SCE_OK;
}

static int check_shape(const sce_shape* s) {
  if (!s) return fail(SCE_EINVAL, "shape is NULL");
  if (s->N <= 0 || s->d <= 0 || s->V <= 0) return fail(SCE_EINVAL, "N, d, V must be positive (got %lld, %lld, %lld)",
                                                       (long long)s->N, (long long)s->d, (long long)s->V);
  if (s->d % 16 != 0) return fail(SCE_EINVAL, "d = %lld must be a multiple of 16", (long long)s->d);
  if (s->N > (1ll << 24) - 256 || s->V > (1ll << 24) - 256 || s->d > (1ll << 24) - 256)
    return fail(SCE_EINVAL, "N, d and V must be below 2^24 (32-bit tile offsets)");
  if (s->V > (int64_t)MAX_SCALE_KBLOCKS * BK)
    return fail(SCE_EINVAL, "V = %lld must be at most %d (the block exponents of a dX tile's K loop wait in LDS)", (long long)s->V, MAX_SCALE_KBLOCKS * BK);
  if (s->d > (1ll << 22) - 256) return fail(SCE_EINVAL, "d = %lld must be below 2^22 (a grid dimension of the layout kernels)", (long long)s->d);
  if (s->n_predict < 1 || s->n_predict > 4) return fail(SCE_EINVAL, "n_predict = %d must be between 1 and 4", s->n_predict);
  return SCE_OK;
}

static size_t sort_tmp_bytes(int64_t N, int64_t V) {
  size_t bytes = 0;
  int bits = 1;
  while ((1ll << bits) <= V) ++bits;
  (void)sce::sort_pairs(nullptr, &bytes, nullptr, nullptr, nullptr, nullptr, (size_t)N, bits, nullptr);
  return bytes;
}

// fp32 partial sums of a K-split dX panel: at most 256 tiles of 256 x 256
constexpr size_t DX_PART_BYTES = (size_t)256 * 256 * 256 * 4;

// The last round of dW tiles, when it is far from full, is shared out along K among DW_TAIL_WGS workgroups
// (bwd_dw_tail_kernel); each leaves its piece of a tile as a 256 x 256 fp32 partial.  A workgroup's range can end inside
// one tile and go on in the next, so there are fewer pieces than workgroups plus tiles.
constexpr int DW_TAIL_WGS = 256;
struct DwTailPlan {
  int full, ntail, kp, share;      // tiles in full rounds, tiles of the last round, pairs of K blocks per tile and per workgroup
  bool use;                        // measured: worth it when the shared-out round is at most half a tile long per workgroup
  size_t bytes;                    // partial tiles: one per (workgroup, tile it touches)
};
static DwTailPlan dw_tail_plan(int64_t dq, int64_t Vp, int64_t krows) {
  DwTailPlan t;
  const int tiles = (int)((dq / 256) * (Vp / 256));
  t.kp = (int)(krows / BK / 2);
  t.full = tiles / DW_TAIL_WGS * DW_TAIL_WGS;
  t.ntail = tiles - t.full;
  t.share = t.ntail > 0 ? (int)(((int64_t)t.ntail * t.kp + DW_TAIL_WGS - 1) / DW_TAIL_WGS) : 0;
  t.use = t.ntail > 0 && t.share >= 1 && t.share * 2 <= t.kp;
  t.bytes = t.use ? (size_t)(DW_TAIL_WGS + t.ntail) * 256 * 256 * 4 : 0;
  return t;
}

// kept: the dlogits come with `saved` (the forward pass emitted them): no panel scratch here
static BwdLayout bwd_layout(const SavedLayout& S, int64_t P, int64_t Pw, int nparts, int K, bool kept = false) {
  BwdLayout B;
  B.P = P; B.Pw = Pw; B.nparts = nparts;
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t r = o; o += (bytes + 255) / 256 * 256; return r; };
  B.off_rho = take((size_t)S.Np * 4);
  B.off_rowinfo = take((size_t)S.Np * 4 * ROWINFO_PLANES);
  B.off_hcoef = take((size_t)S.Np * 4 * K);
  B.off_blockmax = take((size_t)(S.Np / 256) * 4);
  B.off_xi = take(256);
  B.off_xt = take((size_t)S.dq * S.Np);
  B.off_perm = take((size_t)S.N * K * 4 * 2);  // sorted values + unsorted values, one entry per (offset, row)
  B.off_keys = take((size_t)S.N * K * 4 * 2);  // sorted keys + unsorted keys
  B.off_segoff = take((size_t)(S.V + 2) * 4);
  B.off_longlist = take((size_t)(2 * (S.N * K / LONG_SEG + 1) + 2) * 4);   // (column, chunk) pairs: at most one per LONG_SEG entries
  B.off_longbase = take((size_t)S.V * 4);                                  // first slot of each long column
  B.off_longsum = take((size_t)(S.N * K / LONG_SEG + 1) * S.dq * 4);      // chunk sums: a long column has at most one chunk per LONG_SEG of its entries
  B.sorttmp_bytes = sort_tmp_bytes(S.N * K, S.V);
  B.off_sorttmp = take(B.sorttmp_bytes);
  B.off_dxpart = take(DX_PART_BYTES);
  B.fixed = o;
  B.off_ghat_t = take(kept ? 0 : (size_t)S.Vp * Pw);
  B.off_gexp = take(kept ? 0 : (size_t)(S.Vp / 128) * (Pw / 128) * 4);      // block exponents of the dlogits
  B.part_stride = ((size_t)S.dq * S.Vp * 4 + 255) / 256 * 256;
  B.off_dwacc = take(B.part_stride * (size_t)nparts);     // fp32 dW partials, one per dW launch
  B.total = o;
  B.off_dwtail = o;
  B.tail_bytes = S.Np <= Pw ? dw_tail_plan(S.dq, S.Vp, S.Np).bytes : 0;       // (one dW launch over all rows, or no K-split)
  return B;
}

// Rows per panel: as many 256-row tiles as give the dX kernel one full round of tiles on the
// 256 CUs (its tile count is (P / 256) * (dq / 256)), capped by the problem size.
static int64_t default_panel(const SavedLayout& S) {
  int64_t rt = 256 / (S.dq / 256);
  if (rt < 1) rt = 1;
  if (rt > 64) rt = 64;
  const int64_t P = rt * 256;
  return S.Np < P ? S.Np : P;
}
// Rows per dW launch: several dX panels are gathered (transposed) before dW runs, so that its
// fp32 accumulator is read and rewritten less often and its K loop is long.
static int64_t default_dw_panel(const SavedLayout& S, int64_t P) {
  int64_t m = 131072 / P;
  if (m < 1) m = 1;
  int64_t Pw = m * P;
  const int64_t cap = round_up(S.Np, P);
  return Pw < cap ? Pw : cap;
}

// One fp32 dW partial per dW launch (plain stores, summed once at the end) as long as there are
// at most 8; beyond that the last buffer is read, added to and rewritten.
static int dw_launches(const SavedLayout& S, int64_t Pw) {
  const int64_t n = (S.Np + Pw - 1) / Pw;
  return (int)(n < 8 ? n : 8);
}

extern "C" int sce_version(void) { return SCE_VERSION; }

extern "C" int64_t sce_test_set_gather_limit(int64_t bytes) {
  return g_gather_limit.exchange(bytes > 0 && bytes < ((int64_t)1 << 32) ? bytes : (int64_t)1 << 32);
}

extern "C" int sce_timing_enable(int on) {
  std::lock_guard<std::mutex> lk(g_timing_mu);
  for (int k = 0; k < SCE_K_COUNT; ++k) {
    for (hipEvent_t e : g_timing.begin[k]) g_timing.pool.push_back(e);
    for (hipEvent_t e : g_timing.end[k]) g_timing.pool.push_back(e);
    g_timing.begin[k].clear(); g_timing.end[k].clear();
    g_timing.ms[k] = 0.0; g_timing.launches[k] = 0;
  }
  g_timing.on = on != 0;
  return SCE_OK;
}

extern "C" int sce_timing_read(sce_timing* out) {
  if (!out) return fail(SCE_EINVAL, "out is NULL");
  std::lock_guard<std::mutex> lk(g_timing_mu);
  for (int k = 0; k < SCE_K_COUNT; ++k) {
    const size_t n = g_timing.end[k].size();
    for (size_t i = 0; i < n; ++i) {
      float ms = 0.f;
      HIP_TRY(hipEventSynchronize(g_timing.end[k][i]));
      HIP_TRY(hipEventElapsedTime(&ms, g_timing.begin[k][i], g_timing.end[k][i]));
      g_timing.ms[k] += ms; g_timing.launches[k] += 1;
      g_timing.pool.push_back(g_timing.begin[k][i]); g_timing.pool.push_back(g_timing.end[k][i]);
    }
    g_timing.begin[k].clear(); g_timing.end[k].clear();
    out->ms[k] = g_timing.ms[k]; out->launches[k] = g_timing.launches[k];
  }
  return SCE_OK;
}
extern "C" const char* sce_last_error(void) { return g_err; }

// Forward splits V among S workgroups per row tile (each walks CT / S column tiles).  8 keeps the partial records
// small and gives every workgroup a long walk; more (up to 16) only where 8 would leave the last round of
// workgroups, one per CU, mostly empty.
constexpr int FWD_MAX_SPLITS = 16;
static int fwd_splits(int RT, int CT, int ncu) {
  if (CT <= 8) return CT;
  auto fill = [&](int S) { const int64_t wg = (int64_t)RT * S; return (double)wg / (double)((wg + ncu - 1) / ncu * ncu); };
  int best = 8;
  for (int S = 9; S <= FWD_MAX_SPLITS && S <= CT; ++S)
    if (fill(S) > fill(best) + 0.03) best = S;
  return best;
}

extern "C" int sce_sizes_for(const sce_shape* shape, sce_sizes* out) {
  if (int rc = check_shape(shape)) return rc;
  if (!out) return fail(SCE_EINVAL, "out is NULL");
  const SavedLayout S = saved_layout(shape->N, shape->d, shape->V, shape->n_predict);
  out->saved_bytes = S.total;
  out->saved_x_bytes = S.x_total;
  out->wcache_bytes = S.w_total;
  out->fwd_workspace_bytes = (size_t)FWD_MAX_SPLITS * S.Np * 16 + 256;
  out->bwd_workspace_min_bytes = bwd_layout(S, 256, 256, 1, shape->n_predict).total;
  out->bwd_panel_rows = default_panel(S);
  {
    const int64_t Pw = default_dw_panel(S, out->bwd_panel_rows);
    // (both with room for the partial tiles of a K-split last round of dW, where there is to be one)
    const BwdLayout Bd = bwd_layout(S, out->bwd_panel_rows, Pw, dw_launches(S, Pw), shape->n_predict);
    out->bwd_workspace_bytes = Bd.total + Bd.tail_bytes;
    out->dlogits_bytes = S.g_total;
    const BwdLayout Bk = bwd_layout(S, out->bwd_panel_rows, Pw, dw_launches(S, Pw), shape->n_predict, true);
    out->bwd_workspace_kept_bytes = Bk.total + Bk.tail_bytes;
  }
  out->saved_bf16_bytes = saved_layout(shape->N, shape->d, shape->V, shape->n_predict, 2).total;
  return SCE_OK;
}

static int grid_for(size_t work_items, int per_block) {
  size_t g = (work_items + per_block - 1) / per_block;
  if (g > 65536 * 16) g = 65536 * 16;
  if (g == 0) g = 1;
  return (int)g;
}

static int quantize_impl(const void* src, int32_t src_dtype, void* dst, float inv_scale, const float* scale_dev, size_t n, int32_t device,
                         void* stream) {
  if (!src || !dst) return fail(SCE_EINVAL, "src/dst is NULL");
  if (int rc = check_device(device)) return rc;
  if (n == 0) return SCE_OK;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  hipStream_t st = (hipStream_t)stream;
  const int grid = grid_for((n + 3) / 4, 256);
  if (src_dtype == SCE_F32) quantize_flat_kernel<float><<<grid, 256, 0, st>>>((const float*)src, (uint8_t*)dst, n, inv_scale, scale_dev);
  else if (src_dtype == SCE_BF16) quantize_flat_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)src, (uint8_t*)dst, n, inv_scale, scale_dev);
  else return fail(SCE_EINVAL, "unsupported dtype %d", src_dtype);
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

extern "C" int sce_quantize_e4m3(const void* src, int32_t src_dtype, void* dst, double scale, size_t n, int32_t device,
                                 void* stream) {
  if (!(scale > 0.0)) return fail(SCE_EINVAL, "scale must be positive");
  return quantize_impl(src, src_dtype, dst, (float)(1.0 / scale), nullptr, n, device, stream);
}

extern "C" int sce_quantize_e4m3_dev(const void* src, int32_t src_dtype, void* dst, const float* scale_dev, size_t n, int32_t device,
                                     void* stream) {
  if (!scale_dev) return fail(SCE_EINVAL, "scale_dev is NULL");
  return quantize_impl(src, src_dtype, dst, 0.f, scale_dev, n, device, stream);
}

extern "C" int sce_amax_scale(const void* src, int32_t src_dtype, size_t n, float* scale_out, int32_t device, void* stream) {
  if (!src || !scale_out) return fail(SCE_EINVAL, "src/scale_out is NULL");
  if (n == 0) return fail(SCE_EINVAL, "n must be positive");
  if (src_dtype != SCE_F32 && src_dtype != SCE_BF16) return fail(SCE_EINVAL, "unsupported dtype %d", src_dtype);
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  hipStream_t st = (hipStream_t)stream;
  uint32_t* bits = reinterpret_cast<uint32_t*>(scale_out);
  int grid = grid_for(n, 256 * 16);
  if (grid > 4096) grid = 4096;
  amax_begin_kernel<<<1, 1, 0, st>>>(bits);
  if (src_dtype == SCE_F32) amax_kernel<float><<<grid, 256, 0, st>>>((const float*)src, n, bits);
  else amax_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)src, n, bits);
  amax_end_kernel<<<1, 1, 0, st>>>(bits);
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

extern "C" int sce_transpose_bytes(const void* src, void* dst, int64_t rows, int64_t cols, int32_t device, void* stream) {
  if (!src || !dst) return fail(SCE_EINVAL, "src/dst is NULL");
  if (rows <= 0 || cols <= 0) return fail(SCE_EINVAL, "rows and cols must be positive");
  if ((rows + 63) / 64 > 65535) return fail(SCE_EINVAL, "too many rows (%lld)", (long long)rows);
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  transpose_bytes_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)src, (uint8_t*)dst, rows, cols);
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

// own_scratch: the call brings its own scratch (sce_forward_noalloc): args->workspace is not looked at
static int check_common(const sce_args* a, bool own_scratch = false) {
  if (!a) return fail(SCE_EINVAL, "args is NULL");
  if (a->struct_size != sizeof(sce_args)) return fail(SCE_EINVAL, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(sce_args));
  if (int rc = check_shape(&a->shape)) return rc;
  if (!a->targets) return fail(SCE_EINVAL, "targets is NULL");
  if (!(a->cap > 0.f) || a->cap > 40.f) return fail(SCE_EINVAL, "cap = %g must be in (0, 40]", (double)a->cap);
  if (a->operand_dtype == 0 && ((!a->x_s_dev && !(a->x_s > 0.0)) || (!a->w_s_dev && !(a->w_s > 0.0))))
    return fail(SCE_EINVAL, "x_s and w_s must be positive");
  if (a->reduction != SCE_REDUCE_NONE && a->reduction != SCE_REDUCE_MEAN) return fail(SCE_EINVAL, "bad reduction %d", a->reduction);
  if (!a->saved) return fail(SCE_EINVAL, "saved is NULL");
  if (((uintptr_t)a->saved & 255) || (!own_scratch && ((uintptr_t)a->workspace & 255)) || ((uintptr_t)a->wcache & 255))
    return fail(SCE_EINVAL, "saved, workspace and wcache must be 256-byte aligned");
  if (a->vocab_limit < 0 || a->vocab_limit > a->shape.V) return fail(SCE_EINVAL, "vocab_limit must be in [0, V]");
  return check_device(a->device);
}

// ws: the partial records of the V-splits (the caller's workspace, or the library's static scratch)
static int forward_impl(const sce_args* a, void* ws, size_t ws_bytes, const char* ws_name) {
  const int64_t N = a->shape.N, d = a->shape.d, V = a->shape.V;
  if (!a->x || !a->w) return fail(SCE_EINVAL, "x or w is NULL");
  if (a->x_ld < d || a->w_ld < V) return fail(SCE_EINVAL, "row strides smaller than the row length");
  if (a->reduction == SCE_REDUCE_NONE && !a->losses) return fail(SCE_EINVAL, "losses is NULL with reduction = none");
  if (a->reduction == SCE_REDUCE_MEAN && !a->loss) return fail(SCE_EINVAL, "loss is NULL with reduction = mean");
  if (a->reduction == SCE_REDUCE_MEAN && a->shape.n_predict != 1)
    return fail(SCE_EINVAL, "reduction = mean is defined for a single offset only; use reduction = none with n_predict > 1");
  const bool bf16ops = a->operand_dtype == SCE_BF16;
  if (a->operand_dtype != 0 && !bf16ops) return fail(SCE_EINVAL, "operand_dtype %d: 0 (e4m3) or SCE_BF16", a->operand_dtype);
  if (bf16ops && (a->dlogits_from_forward || a->norm || a->wcache))
    return fail(SCE_EINVAL, "bf16 operands are for the forward-only eval head: no kept dlogits, fused norm or weight cache");
  const SavedLayout S = saved_layout(N, d, V, a->shape.n_predict, bf16ops ? 2 : 1);
  const size_t need_saved = a->wcache ? S.x_total : S.total;
  if (a->saved_bytes < need_saved) return fail(SCE_EINVAL, "saved buffer too small: %zu < %zu", a->saved_bytes, need_saved);
  if (a->wcache && a->wcache_bytes < S.w_total) return fail(SCE_EINVAL, "weight cache too small: %zu < %zu", a->wcache_bytes, S.w_total);
  const int64_t Vl = a->vocab_limit > 0 ? a->vocab_limit : V;       // columns that take part
  const int RT = (int)(S.Np / 256), CT = (int)((Vl + 255) / 256);
  const size_t gneed = need_saved + (a->dlogits_from_forward ? S.g_total : 0);
  if (a->saved_bytes < gneed) return fail(SCE_EINVAL, "saved buffer too small for the dlogits: %zu < %zu", a->saved_bytes, gneed);
  DeviceGuard guard(a->device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", a->device);
  (void)hipGetLastError();          // an error left by some earlier, unrelated call is not this call's
  hipStream_t st = (hipStream_t)a->stream;
  uint8_t* sv = (uint8_t*)a->saved;
  uint8_t* xq = sv + S.off_xq;
  uint8_t* wbase = a->wcache ? (uint8_t*)a->wcache : sv + S.x_total;
  uint8_t* wqt = wbase + S.rel_wqt;
  uint8_t* wq = wbase + S.rel_wq;
  uint8_t* gbase = sv + need_saved;       // dlogits, when the forward pass emits them

  // a scale that lives on the device: its value and what follows from it go into the header of `saved`, for the
  // kernels of this call and of the matching backward
  const bool devsc = a->x_s_dev || a->w_s_dev;
  DevConsts* dcp = devsc ? (DevConsts*)(sv + S.off_hdr + 32) : nullptr;
  const float inv_xs = a->x_s_dev ? 0.f : (float)(1.0 / a->x_s), inv_ws = a->w_s_dev ? 0.f : (float)(1.0 / a->w_s);
  {
    KernelTimer tm(SCE_K_QUANT, st);
    if (bf16ops) {
      const int grid = grid_for((size_t)S.Np * (S.dp / 16), 256);
      if (a->x_dtype == SCE_F32) prep_x_bf16_kernel<float><<<grid, 256, 0, st>>>((const float*)a->x, a->x_ld, N, d, (uint16_t*)xq, S.Np, S.dp / 2, S.ldx / 2);
      else if (a->x_dtype == SCE_BF16) prep_x_bf16_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)a->x, a->x_ld, N, d, (uint16_t*)xq, S.Np, S.dp / 2, S.ldx / 2);
      else return fail(SCE_EINVAL, "unsupported x dtype %d", a->x_dtype);
      dim3 gw((unsigned)(S.Vp / 64), (unsigned)(S.dp / 2 / 64));
      if (a->w_dtype == SCE_F32) prep_w_bf16_kernel<float><<<gw, 256, 0, st>>>((const float*)a->w, a->w_ld, d, V, (uint16_t*)wqt, S.ldx / 2);
      else if (a->w_dtype == SCE_BF16) prep_w_bf16_kernel<bf16_t><<<gw, 256, 0, st>>>((const bf16_t*)a->w, a->w_ld, d, V, (uint16_t*)wqt, S.ldx / 2);
      else return fail(SCE_EINVAL, "unsupported w dtype %d", a->w_dtype);
    }
    if (devsc && !bf16ops) dev_consts_kernel<<<1, 1, 0, st>>>(a->x_s_dev, a->w_s_dev, (float)a->x_s, (float)a->w_s, a->cap, dcp);
    const int grid = grid_for((size_t)S.Np * (S.dp / 16), 256);
    float* rstd = (float*)(sv + S.off_rstd);
    const int ngrid = (int)((S.Np + 3) / 4);
    if (bf16ops) {
      // operands laid out above
    } else if (a->norm && a->x_dtype == SCE_F32)
      rmsnorm_quantize_kernel<float><<<ngrid, 256, 0, st>>>((const float*)a->x, a->x_ld, N, d, a->norm_eps, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev, rstd);
    else if (a->norm && a->x_dtype == SCE_BF16)
      rmsnorm_quantize_kernel<bf16_t><<<ngrid, 256, 0, st>>>((const bf16_t*)a->x, a->x_ld, N, d, a->norm_eps, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev, rstd);
    else if (a->x_dtype == SCE_F32)
      quantize_pad_kernel<float><<<grid, 256, 0, st>>>((const float*)a->x, a->x_ld, N, d, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev);
    else if (a->x_dtype == SCE_BF16)
      quantize_pad_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)a->x, a->x_ld, N, d, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev);
    else return fail(SCE_EINVAL, "unsupported x dtype %d", a->x_dtype);
    dim3 gw((unsigned)(S.Vp / QW_TILE), (unsigned)(S.dq / QW_TILE));
    if (bf16ops) {
    } else if (a->wcache && a->wcache_valid) {
      // the caller vouches that the cache holds e4m3(W / w_s) of this W (unchanged since an earlier call)
    } else if (a->w_dtype == SCE_F32)
      quantize_w_kernel<float><<<gw, 256, 0, st>>>((const float*)a->w, a->w_ld, d, V, wq, wqt, S.dp, S.ldx, S.Vp / BK, inv_ws, a->w_s_dev);
    else if (a->w_dtype == SCE_BF16)
      quantize_w_kernel<bf16_t><<<gw, 256, 0, st>>>((const bf16_t*)a->w, a->w_ld, d, V, wq, wqt, S.dp, S.ldx, S.Vp / BK, inv_ws, a->w_s_dev);
    else return fail(SCE_EINVAL, "unsupported w dtype %d", a->w_dtype);
  }
  const bool emit = a->dlogits_from_forward != 0;
  const int CTw = emit ? (int)(S.Vp / 256) : CT;       // with the dlogits every tile is visited: the masked ones must read as zero later
  const int nsplit = fwd_splits(RT, CTw, device_cus_or_default(a->device));
  const size_t need_ws = (size_t)nsplit * S.Np * 16;
  if (!ws || ws_bytes < need_ws) return fail(SCE_EINVAL, "%s too small: %zu < %zu", ws_name, ws_bytes, need_ws);
  FwdParams p;
  p.xq = xq; p.wqt = wqt; p.partials = (float4*)ws;
  p.targets = a->targets; p.ignore_index = a->ignore_index; p.n_predict = a->shape.n_predict; p.s_uy = (float*)(sv + S.off_zy);
  p.ghat_t = emit ? gbase + S.rel_g : nullptr; p.gexp = emit ? (uint32_t*)(gbase + S.rel_gexp) : nullptr; p.kbw = S.Np / BK; p.kbv = S.Vp / BK;
  p.dp = S.dp; p.ldx = S.ldx; p.N = (int)N; p.V = (int)Vl; p.Np = (int)S.Np; p.RT = RT; p.CT = CTw; p.S = nsplit;
  p.sc = bf16ops ? 1.0f : (float)a->x_s * (float)a->w_s; p.k1 = p.sc * 2.0f * LOG2E / a->cap; p.c2 = -2.0f * a->cap * LOG2E; p.ic2 = 1.0f / p.c2; p.em2cap = expf(-2.0f * a->cap);
  p.dc = bf16ops ? nullptr : dcp;
  p.want_argmax = a->argmax != nullptr;
  const int grid = 8 * nsplit * ((RT + 7) / 8);
  // An fp8 forward pass has its target logits computed ahead of the forward kernel (from a tile of gathered rows of W_q^T,
  // together with the rows' boosts when it emits the dlogits) as long as that tile's 32-bit offsets reach every row of
  // W_q^T; beyond, the forward kernel takes them out of its own accumulators, as the bf16 forward pass does.
  const bool pre = !bf16ops && (int64_t)S.Vp * S.ldx < g_gather_limit;
  {
    // the exponent boosts of the rows, estimated from two tiles of their logits: only for a forward pass
    // that emits the dlogits (a backward pass that forms them again knows the rows' sums and takes the boosts from those)
    KernelTimer tm(SCE_K_QUANT, st);
    float* lam = (float*)(sv + S.off_lam);
    p.lam = lam;
    if (!bf16ops && emit) {
      if (pre) fwd_sample_kernel<true><<<RT, NTHREADS, SMEM_SAMPLE, st>>>(p, CT / 2, lam);
      else fwd_sample_kernel<false><<<RT, NTHREADS, SMEM_SAMPLE, st>>>(p, CT / 2, lam);
    } else if (pre) fwd_sample_kernel<true, false><<<RT, NTHREADS, SMEM_SAMPLE, st>>>(p, CT / 2, lam);
  }
  {
    KernelTimer tm(SCE_K_FWD, st);
    if (emit && pre) {
      fwd_kernel<true, false, true><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
      fwd_knock_kernel<<<(int)(S.Np / 256), 256, 0, st>>>(p.ghat_t, p.kbv, a->targets, a->ignore_index, (int)N, (int)Vl, a->shape.n_predict);
    } else if (emit) fwd_kernel<true><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
    else if (bf16ops) fwd_kernel<false, true><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
    else if (pre) fwd_kernel<false, false, true><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
    else fwd_kernel<false><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
  }
  KernelTimer tm_red(SCE_K_FWD_REDUCE, st);
  float* s_lse = (float*)(sv + S.off_lse);
  float* s_umax = (float*)(sv + S.off_umax);
  float* s_zy = (float*)(sv + S.off_zy);
  fwd_combine_kernel<<<(int)(S.Np / 256), 256, 0, st>>>(p.partials, nsplit, (int)N, (int)S.Np, (int)Vl, a->targets, a->ignore_index,
                                                       a->cap, a->mtp_weights, a->shape.n_predict, s_lse, s_umax, s_zy, a->losses, a->lse,
                                                       a->argmax);
  fwd_reduce_kernel<<<1, 1024, 0, st>>>(p.partials, (int)(S.Np / 256), (int32_t*)(sv + S.off_hdr),
                                        a->reduction == SCE_REDUCE_MEAN ? a->loss : nullptr, a->n_valid,
                                        call_mode(emit, (int)Vl, a->shape.n_predict, a->cap));
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

extern "C" int sce_forward(const sce_args* a) {
  if (int rc = check_common(a)) return rc;
  return forward_impl(a, a->workspace, a->workspace_bytes, "forward workspace");
}

// The same launches as sce_forward with the partial records in the library's static device array instead of a
// caller's workspace: no allocation, by the caller for this call or by the library ever.  Calls on one device share
// the array; nothing in it has to start at zero (the forward kernel writes every record that the combine kernel
// reads), so nothing is cleared, but two calls in flight on one device at a time would overwrite each other's records.
extern "C" int sce_forward_noalloc(const sce_args* a) {
  if (int rc = check_common(a, true)) return rc;
  void* sp = g_scratch[a->device];              // set by check_device (inside check_common) for this very device
  if (!sp) return fail(SCE_EHIP, "no static scratch on device %d", a->device);
  return forward_impl(a, sp, NOALLOC_SCRATCH_BYTES,
                      "the static scratch of sce_forward_noalloc (8 MiB: N rounded up to 256 times the number of V-splits, 8 to 16, "
                      "may not exceed 524288; use sce_forward with a workspace)");
}

extern "C" int sce_backward(const sce_args* a) {
  if (int rc = check_common(a)) return rc;
  const int64_t N = a->shape.N, d = a->shape.d, V = a->shape.V;
  if (a->operand_dtype != 0) return fail(SCE_EINVAL, "bf16 operands are forward only (the eval head)");
  if (!a->grad_output) return fail(SCE_EINVAL, "grad_output is NULL");
  if (!a->dx || !a->dw) return fail(SCE_EINVAL, "dx or dw is NULL");
  if (a->norm) {
    if (!a->x) return fail(SCE_EINVAL, "norm is set: backward needs x (the hidden state given to forward)");
    if (a->x_dtype != SCE_F32 && a->x_dtype != SCE_BF16) return fail(SCE_EINVAL, "unsupported x dtype %d", a->x_dtype);
    if (a->x_ld < d) return fail(SCE_EINVAL, "row strides smaller than the row length");
  }
  if (a->dx_ld < d || a->dw_ld < V) return fail(SCE_EINVAL, "row strides smaller than the row length");
  if ((a->dx_dtype != SCE_F32 && a->dx_dtype != SCE_BF16) || (a->dw_dtype != SCE_F32 && a->dw_dtype != SCE_BF16))
    return fail(SCE_EINVAL, "unsupported gradient dtype");
  const SavedLayout S = saved_layout(N, d, V, a->shape.n_predict);
  const size_t need_saved = a->wcache ? S.x_total : S.total;
  if (a->saved_bytes < need_saved) return fail(SCE_EINVAL, "saved buffer too small: %zu < %zu", a->saved_bytes, need_saved);
  if (a->wcache && a->wcache_bytes < S.w_total) return fail(SCE_EINVAL, "weight cache too small: %zu < %zu", a->wcache_bytes, S.w_total);
  const int64_t Vl = a->vocab_limit > 0 ? a->vocab_limit : V;       // columns that take part
  if (!a->workspace) return fail(SCE_EINVAL, "workspace is NULL");
  const int K = a->shape.n_predict;
  const bool kept = a->dlogits_from_forward != 0;        // the dlogits came with `saved`
  if (kept && a->saved_bytes < need_saved + S.g_total)
    return fail(SCE_EINVAL, "saved buffer too small for the dlogits: %zu < %zu", a->saved_bytes, need_saved + S.g_total);
  const BwdLayout Bmin = bwd_layout(S, 256, 256, 1, K, kept);
  if (a->workspace_bytes < Bmin.total) return fail(SCE_EINVAL, "backward workspace too small: %zu < %zu", a->workspace_bytes, Bmin.total);
  if (a->panel_rows % 256) return fail(SCE_EINVAL, "panel_rows must be a multiple of 256");
  // panel sizes from what the caller gave: P rows per recompute/dX panel, Pw = m * P rows per dW launch
  int64_t P, Pw;
  int nparts;
  if (kept) {
    // dX still goes panel by panel, one round of tiles each: a launch with several rounds was measured 2 % slower
    P = a->panel_rows > 0 ? a->panel_rows : default_panel(S);
    if (P > S.Np) P = S.Np;
    if (P > 131072) P = 131072;
    Pw = default_dw_panel(S, P);
    nparts = dw_launches(S, Pw);
    while (nparts > 1 && bwd_layout(S, P, Pw, nparts, K, true).total > a->workspace_bytes) --nparts;
  } else {
    // bytes left for the e4m3 dlogits: Vp rows of Pw bytes
    const int64_t room = (int64_t)(a->workspace_bytes - Bmin.fixed - Bmin.part_stride);
    P = default_panel(S);
    if (a->panel_rows > 0) {
      P = a->panel_rows < S.Np ? a->panel_rows : S.Np;
      if (P > 131072) P = 131072;          // a dW launch covers at least one panel and at most MAX_SCALE_KBLOCKS K blocks
    }
    if (P * S.Vp > room) P = room / S.Vp / 256 * 256;
    if (P < 256) P = 256;                                  // Bmin fits, as checked above
    Pw = default_dw_panel(S, P);
    if (Pw * S.Vp > room) Pw = room / S.Vp / P * P;
    if (Pw < P) Pw = P;
    nparts = dw_launches(S, Pw);
    // the estimate above ignores the 256-byte alignment of each region: settle on a layout that fits
    while (bwd_layout(S, P, Pw, nparts, K).total > a->workspace_bytes) {
      if (nparts > 1) --nparts;
      else if (Pw > P) Pw -= P;
      else if (P > 256) { P -= 256; Pw = P; }
      else return fail(SCE_EINVAL, "internal: panel layout exceeds workspace");
    }
  }
  const BwdLayout B = bwd_layout(S, P, Pw, nparts, K, kept);
  DeviceGuard guard(a->device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", a->device);
  (void)hipGetLastError();          // an error left by some earlier, unrelated call is not this call's
  hipStream_t st = (hipStream_t)a->stream;
  uint8_t* sv = (uint8_t*)a->saved;
  uint8_t* ws = (uint8_t*)a->workspace;
  const uint8_t* xq = sv + S.off_xq;
  const uint8_t* wbase = a->wcache ? (const uint8_t*)a->wcache : sv + S.x_total;
  const uint8_t* wqt = wbase + S.rel_wqt;
  const uint8_t* wq = wbase + S.rel_wq;
  const float* s_lse = (const float*)(sv + S.off_lse);
  const float* s_zy = (const float*)(sv + S.off_zy);
  const int32_t* hdr = (const int32_t*)(sv + S.off_hdr);
  const DevConsts* dcp = (a->x_s_dev || a->w_s_dev) ? (const DevConsts*)(sv + S.off_hdr + 32) : nullptr;     // as forward left it
  uint8_t* gkept = sv + need_saved;
  uint32_t* gexp = kept ? (uint32_t*)(gkept + S.rel_gexp) : (uint32_t*)(ws + B.off_gexp);
  float* rho = (float*)(ws + B.off_rho);
  int32_t* rowinfo = (int32_t*)(ws + B.off_rowinfo);
  float* hcoef = (float*)(ws + B.off_hcoef);
  float* blockmax = (float*)(ws + B.off_blockmax);
  float* xi = (float*)(ws + B.off_xi);
  uint8_t* xt = ws + B.off_xt;
  float* dwacc = (float*)(ws + B.off_dwacc);
  int32_t* perm = (int32_t*)(ws + B.off_perm);
  const int64_t NE = N * K;            // one-hot entries: one per (offset, row)
  int32_t* vals_in = perm + NE;
  int32_t* skeys = (int32_t*)(ws + B.off_keys);
  int32_t* keys_in = skeys + NE;
  int32_t* segoff = (int32_t*)(ws + B.off_segoff);
  int32_t* longlist = (int32_t*)(ws + B.off_longlist);
  float* longsum = (float*)(ws + B.off_longsum);
  int32_t* longbase = (int32_t*)(ws + B.off_longbase);
  uint8_t* ghat_t = kept ? gkept + S.rel_g : ws + B.off_ghat_t;
  const int64_t gkb = kept ? S.Np / BK : Pw / BK;      // K blocks per v tile of the dlogits buffer

  const int nblk = (int)(S.Np / 256);
  KernelTimer* tm_prep = new KernelTimer(SCE_K_BWD_PREP, st);
  bwd_prep_kernel<<<nblk, 256, 0, st>>>(s_lse, s_zy, a->targets, a->ignore_index, hdr, a->grad_output,
                                        a->reduction == SCE_REDUCE_NONE ? 1 : 0, a->grad_scale, a->mtp_weights, K, a->cap, (int)N,
                                        (int)S.Np, (int)Vl, (const float*)(sv + S.off_lam), rho, hcoef, blockmax, kept ? nullptr : rowinfo,
                                        call_mode(kept, (int)Vl, K, a->cap));
  bwd_xi_kernel<<<1, 1024, 0, st>>>(blockmax, nblk, xi);
  {
    dim3 g((unsigned)(S.Np / XT_TILE), (unsigned)(S.dq / XT_TILE));
    bwd_xt_kernel<<<g, 256, 0, st>>>(xq, S.dp, S.ldx, S.Np / BK, rho, xi, xt);
  }
  // rows grouped by target, for the one-hot part of dW
  {
    bwd_keys_kernel<<<(int)((NE + 255) / 256), 256, 0, st>>>(a->targets, a->ignore_index, (int)N, (int)S.Np, (int)Vl, (int)V, K, keys_in, vals_in, longlist);
    int bits = 1;
    while ((1ll << bits) <= V) ++bits;
    size_t tmp = B.sorttmp_bytes;
    if (sce::sort_pairs(ws + B.off_sorttmp, &tmp, keys_in, skeys, vals_in, perm, (size_t)NE, bits, st) != 0)
    { delete tm_prep; return fail(SCE_EHIP, "radix sort of the targets failed"); }
    bwd_segoff_kernel<<<(int)((NE + 256) / 256), 256, 0, st>>>(skeys, (int)NE, (int)V, segoff);
    bwd_longlist_kernel<<<(int)((V + 255) / 256), 256, 0, st>>>(segoff, (int)V, longlist, longbase);
  }
  delete tm_prep;
  const float sc = (float)a->x_s * (float)a->w_s, k1 = sc * 2.0f * LOG2E / a->cap, c2 = -2.0f * a->cap * LOG2E;
  const int CTv = (int)(S.Vp / 256), CTd = (int)(S.dq / 256);
  int launch = 0;
  DwTail tail;
  tail.buf = nullptr; tail.tile0 = -1; tail.ntail = 0; tail.kp = 1; tail.share = 1;
  const bool dx_f32 = a->dx_dtype == SCE_F32;
  const int smem_dx = smem_scaled((int)(S.Vp / BK), SMEM_DX);
  // dX of the rows [p0, p0 + prow) (a multiple of 256), the dlogits buffer standing for rows from gorg on
  auto dx_params = [&](int64_t p0, int64_t prow, int64_t gorg) {
    DxParams q;
    q.wq = wq; q.ghat_t = ghat_t + ((p0 - gorg) / 256) * (S.Vp / BK) * BLOCKED_KSTEP; q.gexp = gexp + (p0 - gorg) / BK; q.kbw = gkb; q.wqt = wqt; q.rho = rho + p0; q.hcoef = hcoef + p0; q.targets = a->targets + p0;
    q.dx_ld = a->dx_ld; q.Vp = S.Vp; q.ldx = S.ldx; q.Np = S.Np; q.dq = S.dq; q.RT = (int)(prow / 256); q.CT = CTd;
    q.n_predict = K; q.rows_left = (int)(N - p0 > 0 ? N - p0 : 0);
    q.rows = (int)((N - p0 < prow) ? (N - p0 > 0 ? N - p0 : 0) : prow); q.d = (int)d; q.V = (int)Vl; q.w_s = (float)a->w_s; q.dc = dcp;
    q.part = (float*)(ws + B.off_dxpart);
    q.ksplit = 1;
    q.dx = dx_f32 ? (void*)((float*)a->dx + p0 * a->dx_ld) : (void*)((bf16_t*)a->dx + p0 * a->dx_ld);
    return q;
  };
  auto dx_panel = [&](int64_t p0, int64_t prow, int64_t gorg) {
    DxParams dp_ = dx_params(p0, prow, gorg);
    // a panel with fewer than half as many tiles as there are CUs shares each tile's K loop among several workgroups
    const int tiles = dp_.RT * CTd, kpairs = (int)(S.Vp / BK / 2);
    int ksplit = tiles * 2 <= 256 ? 256 / tiles : 1;
    if (ksplit > 8) ksplit = 8;
    if (ksplit > kpairs) ksplit = kpairs;
    dp_.ksplit = ksplit;
    KernelTimer tm(SCE_K_DX, st);
    if (ksplit == 1) {
      if (dx_f32) bwd_dx_kernel<float, false><<<map_tile_grid(dp_.RT, CTd), NTHREADS, smem_dx, st>>>(dp_);
      else bwd_dx_kernel<bf16_t, false><<<map_tile_grid(dp_.RT, CTd), NTHREADS, smem_dx, st>>>(dp_);
    } else if (dp_.rows > 0) {
      const int fgrid = (int)(((int64_t)dp_.rows * (d / 4) + 255) / 256);
      if (dx_f32) {
        bwd_dx_kernel<float, true><<<map_tile_grid(dp_.RT, CTd * ksplit), NTHREADS, smem_dx, st>>>(dp_);
        bwd_dx_finish_kernel<float><<<fgrid, 256, 0, st>>>(dp_);
      } else {
        bwd_dx_kernel<bf16_t, true><<<map_tile_grid(dp_.RT, CTd * ksplit), NTHREADS, smem_dx, st>>>(dp_);
        bwd_dx_finish_kernel<bf16_t><<<fgrid, 256, 0, st>>>(dp_);
      }
    }
  };
  // dW over the rows [w0, w0 + gathered)
  auto dw_launch = [&](int64_t w0, int64_t gathered, int64_t gorg, bool last) {
    DwParams wp;
    const int part = launch < nparts ? launch : nparts - 1;
    wp.xt = xt; wp.ghat_t = ghat_t + ((w0 - gorg) / 256) * (S.Vp / BK) * BLOCKED_KSTEP; wp.gexp = gexp + (w0 - gorg) / BK; wp.dwacc = (float*)((uint8_t*)dwacc + (size_t)part * B.part_stride);
    wp.kbn = S.Np / BK; wp.kbw = gkb; wp.kb0 = w0 / BK; wp.Vp = S.Vp; wp.kbv = S.Vp / BK;
    wp.RT = CTd; wp.CT = CTv; wp.KT = (int)(gathered / BK);
    {
      KernelTimer tm(SCE_K_DW, st);
      // When this launch is the only one and its last round of tiles would leave many CUs idle, that round is
      // shared out along K instead (bwd_dw_tail_kernel): the full rounds run as they are.
      const DwTailPlan tp = dw_tail_plan(S.dq, S.Vp, gathered);
      const bool only = w0 == 0 && last && launch == 0;
      if (only && tp.use && B.tail_bytes >= tp.bytes && a->workspace_bytes >= B.off_dwtail + tp.bytes) {
        const int full = tp.full;
        tail.buf = (float*)(ws + B.off_dwtail); tail.tile0 = tp.full; tail.ntail = tp.ntail; tail.kp = tp.kp; tail.share = tp.share;
        if (full > 0) bwd_dw_kernel<false><<<full, NTHREADS, smem_scaled(wp.KT, 0), st>>>(wp);
        bwd_dw_tail_kernel<<<dim3(DW_TAIL_WGS, 2), NTHREADS, smem_scaled(2 * tp.share, 0), st>>>(wp, tail);
      } else if (launch >= nparts) bwd_dw_kernel<true><<<map_tile_rr_grid(CTd, CTv), NTHREADS, smem_scaled(wp.KT, 0), st>>>(wp);
      else bwd_dw_kernel<false><<<map_tile_rr_grid(CTd, CTv), NTHREADS, smem_scaled(wp.KT, 0), st>>>(wp);
    }
    ++launch;
  };
  if (kept) {
    // The dlogits of all rows are there: dX and dW are independent of each other.  dX still goes panel by panel, one
    // round of tiles each.  (One grid of tiles over all rows, launched 256 tiles at a time -- ten full rounds at N = 65536,
    // d = 2560 instead of ten panels of 250 tiles and a ragged eleventh -- was measured no faster: a launch of 256 tiles takes
    // 0.58 ms where one of 250 takes 0.56.  Under fp8 MFMA load the part runs at the clock its power limit allows, and
    // compute units left idle leave the others a higher one.)
    for (int64_t p0 = 0; p0 < S.Np; p0 += P) dx_panel(p0, (S.Np - p0 < P) ? (S.Np - p0) : P, 0);
    for (int64_t w0 = 0; w0 < S.Np; w0 += Pw) dw_launch(w0, (S.Np - w0 < Pw) ? (S.Np - w0) : Pw, 0, w0 + Pw >= S.Np);
  } else {
    int64_t w0 = 0;                      // first row of the rows gathered for the next dW launch
    for (int64_t p0 = 0; p0 < S.Np; p0 += P) {
      const int64_t prow = (S.Np - p0 < P) ? (S.Np - p0) : P;     // multiple of 256
      const int RTp = (int)(prow / 256);
      const int64_t gorg = w0;                                    // the row that K block 0 of the dlogits buffer stands for
      RecomputeParams rp;
      rp.xq = xq + p0 * S.ldx; rp.wqt = wqt; rp.ghat_t = ghat_t; rp.gexp = gexp; rp.rowinfo = rowinfo + p0; rp.Np = S.Np; rp.n_predict = K;
      rp.dp = S.dp; rp.ldx = S.ldx; rp.kbw = gkb; rp.kbv = S.Vp / BK; rp.kb0 = (p0 - gorg) / BK; rp.RT = RTp; rp.CT = CTv; rp.V = (int)Vl; rp.k1 = k1; rp.c2 = c2; rp.sc = sc; rp.dc = dcp;
      {
        KernelTimer tm(SCE_K_RECOMPUTE, st);
        bwd_recompute_kernel<<<map_tile_grid(RTp, CTv), NTHREADS, SMEM_RECOMPUTE, st>>>(rp);
        if (p0 < N)       // the target entries of the panel's rows are cleared (rows p0 on: tiles (p0 - gorg) / 256 on of the buffer)
          fwd_knock_kernel<<<(int)(prow / 256), 256, 0, st>>>(ghat_t + (size_t)((p0 - gorg) / 256) * (S.Vp / BK) * BLOCKED_KSTEP, S.Vp / BK, a->targets + p0,
                                                          a->ignore_index, (int)(N - p0), (int)Vl, K);
      }
      dx_panel(p0, prow, gorg);
      const int64_t gathered = p0 + prow - w0;
      if (gathered + P > Pw || p0 + prow >= S.Np) {      // the transposed scratch is full, or this was the last panel
        dw_launch(w0, gathered, gorg, p0 + prow >= S.Np);
        w0 = p0 + prow;
      }
    }
  }
  if (a->norm) {       // dX so far is the gradient of the normalised rows: take it through the norm, in place
    const float* rstd = (const float*)(sv + S.off_rstd);
    const int ngrid = (int)((N + 3) / 4);
    const bool gf = a->dx_dtype == SCE_F32, hf = a->x_dtype == SCE_F32;
    if (gf && hf) rmsnorm_backward_kernel<float, float><<<ngrid, 256, 0, st>>>((float*)a->dx, a->dx_ld, (const float*)a->x, a->x_ld, rstd, N, d);
    else if (gf) rmsnorm_backward_kernel<float, bf16_t><<<ngrid, 256, 0, st>>>((float*)a->dx, a->dx_ld, (const bf16_t*)a->x, a->x_ld, rstd, N, d);
    else if (hf) rmsnorm_backward_kernel<bf16_t, float><<<ngrid, 256, 0, st>>>((bf16_t*)a->dx, a->dx_ld, (const float*)a->x, a->x_ld, rstd, N, d);
    else rmsnorm_backward_kernel<bf16_t, bf16_t><<<ngrid, 256, 0, st>>>((bf16_t*)a->dx, a->dx_ld, (const bf16_t*)a->x, a->x_ld, rstd, N, d);
  }
  KernelTimer tm_fin(SCE_K_DW_FINAL, st);
  bwd_dw_long_kernel<<<dim3((unsigned)(NE / LONG_SEG + 1), (unsigned)(S.dq / 256)), 256, 0, st>>>(longlist, segoff, perm, hcoef, xq, S.dp, S.ldx, S.dq, (int)S.Np, longsum);
  {
    dim3 g((unsigned)((V + 63) / 64), (unsigned)((d + 63) / 64));
    if (a->dw_dtype == SCE_F32)
      bwd_dw_final_kernel<float><<<g, 256, 0, st>>>(dwacc, launch < nparts ? launch : nparts, (int64_t)(B.part_stride / 4), S.Vp, segoff, perm, hcoef, xq, S.ldx, (int)S.Np, xi, longsum, longbase, S.dq, (float)a->x_s, dcp, (int)d, (int)V,
                                                   (float*)a->dw, a->dw_ld, tail, CTd, CTv);
    else
      bwd_dw_final_kernel<bf16_t><<<g, 256, 0, st>>>(dwacc, launch < nparts ? launch : nparts, (int64_t)(B.part_stride / 4), S.Vp, segoff, perm, hcoef, xq, S.ldx, (int)S.Np, xi, longsum, longbase, S.dq, (float)a->x_s, dcp, (int)d, (int)V,
                                                    (bf16_t*)a->dw, a->dw_ld, tail, CTd, CTv);
  }
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

// ------------------------------------------------------------------------------------------
// measurement aids
// ------------------------------------------------------------------------------------------
struct EventPair {   // two timing events that are destroyed on every way out
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t create() {
    hipError_t e = hipEventCreate(&e0);
    return e != hipSuccess ? e : hipEventCreate(&e1);
  }
  ~EventPair() {
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  }
};

static double median_mhz(const long long* clk, int n) {
  std::vector<double> v;
  for (int i = 0; i < n; ++i)
    if (clk[2 * i + 1] > 0) v.push_back((double)clk[2 * i] / (double)clk[2 * i + 1] * 100.0);
  if (v.empty()) return 0.0;
  std::sort(v.begin(), v.end());
  return v[v.size() / 2];
}

extern "C" int sce_bench_mfma(const void* random_bytes, size_t random_bytes_size, int32_t iters, int32_t reps, void* scratch, size_t scratch_bytes,
                              int32_t device, void* stream, double* tflops, double* shader_mhz) {
  if (!scratch || !tflops || !shader_mhz || iters <= 0 || reps <= 0) return fail(SCE_EINVAL, "bad argument");
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  const int ncu = device_cus_or_default(device), grid = 4 * ncu;           // one wave per SIMD would be grid = ncu; four keep every SIMD fed
  const size_t need = (size_t)grid * 256 * 4 + 2 * 1024 * sizeof(long long);
  if (scratch_bytes < need) return fail(SCE_EINVAL, "scratch too small: %zu < %zu", scratch_bytes, need);
  // every thread of the grid reads 8 fragments of 32 bytes
  const size_t need_random = (size_t)grid * 256 * 8 * 32;
  if (random_bytes && random_bytes_size < need_random)
    return fail(SCE_EINVAL, "random_bytes too small: %zu < %zu (64 KiB for each of 4 workgroups per compute unit)", random_bytes_size, need_random);
  hipStream_t st = (hipStream_t)stream;
  float* out = (float*)scratch;
  long long* clk = (long long*)((uint8_t*)scratch + (size_t)grid * 256 * 4);
  EventPair ev;
  HIP_TRY(ev.create());
  const hipEvent_t e0 = ev.e0, e1 = ev.e1;
  bench_mfma_kernel<<<grid, 256, 0, st>>>((const uint8_t*)random_bytes, iters, out, clk);      // warm-up
  HIP_TRY(hipEventRecord(e0, st));
  for (int r = 0; r < reps; ++r) bench_mfma_kernel<<<grid, 256, 0, st>>>((const uint8_t*)random_bytes, iters, out, clk);
  HIP_TRY(hipEventRecord(e1, st));
  HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  std::vector<long long> h(2 * 1024);
  HIP_TRY(hipMemcpy(h.data(), clk, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
  const double flops = (double)reps * grid * 4.0 * iters * 16.0 * (2.0 * 32 * 32 * 64);
  *tflops = flops / (ms * 1e-3) * 1e-12;
  *shader_mhz = median_mhz(h.data(), grid < 1024 ? grid : 1024);
  return SCE_OK;
}

extern "C" int sce_bench_gemm(const void* A, const void* B, int64_t M, int64_t N, int64_t K, int32_t reps, void* scratch, size_t scratch_bytes,
                              int32_t device, void* stream, double* tflops, double* shader_mhz) {
  if (!A || !B || !scratch || !tflops || !shader_mhz || reps <= 0) return fail(SCE_EINVAL, "bad argument");
  if (M <= 0 || N <= 0 || K <= 0 || M % 256 || N % 256 || K % 256) return fail(SCE_EINVAL, "M, N, K must be positive multiples of 256");
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  const int RT = (int)(M / 256), CT = (int)(N / 256), grid = map_tile_grid(RT, CT);
  const size_t need = (size_t)grid * 256 * 4 + 2 * 1024 * sizeof(long long);
  if (scratch_bytes < need) return fail(SCE_EINVAL, "scratch too small: %zu < %zu", scratch_bytes, need);
  HIP_TRY(hipFuncSetAttribute((const void*)bench_gemm_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES));
  hipStream_t st = (hipStream_t)stream;
  float* out = (float*)scratch;
  long long* clk = (long long*)((uint8_t*)scratch + (size_t)grid * 256 * 4);
  const int64_t ld = row_stride(K);
  EventPair ev;
  HIP_TRY(ev.create());
  const hipEvent_t e0 = ev.e0, e1 = ev.e1;
  bench_gemm_kernel<<<grid, NTHREADS, SMEM_BYTES, st>>>((const uint8_t*)A, (const uint8_t*)B, out, (int)(K / BK), RT, CT, ld, clk);
  HIP_TRY(hipEventRecord(e0, st));
  for (int r = 0; r < reps; ++r)
    bench_gemm_kernel<<<grid, NTHREADS, SMEM_BYTES, st>>>((const uint8_t*)A, (const uint8_t*)B, out, (int)(K / BK), RT, CT, ld, clk);
  HIP_TRY(hipEventRecord(e1, st));
  HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  std::vector<long long> h(2 * 1024);
  HIP_TRY(hipMemcpy(h.data(), clk, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
  *tflops = 2.0 * M * N * K * reps / (ms * 1e-3) * 1e-12;
  *shader_mhz = median_mhz(h.data(), grid < 1024 ? grid : 1024);
  return SCE_OK;
}

// The main loops of the forward, dX and dW kernels alone on the buffers that a forward call with dlogits_from_forward and
// the matching backward call have filled (see include/slowrun_ce.h).
extern "C" int sce_bench_floor(const sce_args* a, int32_t which, int32_t reps, void* scratch, size_t scratch_bytes, double* ms_per_pass,
                               double* shader_mhz) {
  if (int rc = check_common(a)) return rc;
  if (!scratch || !ms_per_pass || !shader_mhz || reps <= 0) return fail(SCE_EINVAL, "bad argument");
  if (which != SCE_K_FWD && which != SCE_K_DX && which != SCE_K_DW) return fail(SCE_EINVAL, "which must be SCE_K_FWD, SCE_K_DX or SCE_K_DW");
  if (!a->dlogits_from_forward || a->operand_dtype != 0 || a->wcache) return fail(SCE_EINVAL, "needs the saved state of a forward call with dlogits_from_forward (e4m3 operands, no weight cache)");
  const int64_t N = a->shape.N, d = a->shape.d, V = a->shape.V;
  const int K = a->shape.n_predict;
  const SavedLayout S = saved_layout(N, d, V, K);
  if (a->saved_bytes < S.total + S.g_total) return fail(SCE_EINVAL, "saved buffer too small: %zu < %zu", a->saved_bytes, S.total + S.g_total);
  if (S.Np > 131072) return fail(SCE_EINVAL, "at most 131072 rows (one dW launch)");
  const int64_t P = default_panel(S);
  const BwdLayout B = bwd_layout(S, P, default_dw_panel(S, P), 1, K, true);
  if (which == SCE_K_DW && (!a->workspace || a->workspace_bytes < B.off_xt + (size_t)S.dq * S.Np)) return fail(SCE_EINVAL, "backward workspace too small");
  HIP_TRY(hipFuncSetAttribute((const void*)floor_fwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES));
  HIP_TRY(hipFuncSetAttribute((const void*)floor_dx_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
  HIP_TRY(hipFuncSetAttribute((const void*)floor_dw_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
  DeviceGuard guard(a->device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", a->device);
  hipStream_t st = (hipStream_t)a->stream;
  const uint8_t* sv = (const uint8_t*)a->saved;
  const uint8_t* xq = sv + S.off_xq;
  const uint8_t* wqt = sv + S.x_total + S.rel_wqt;
  const uint8_t* wq = sv + S.x_total + S.rel_wq;
  const uint8_t* ghat_t = sv + S.total + S.rel_g;
  const uint32_t* gexp = (const uint32_t*)(sv + S.total + S.rel_gexp);
  const int RT = (int)(S.Np / 256), CTv = (int)(S.Vp / 256), CTd = (int)(S.dq / 256);
  const int nsplit = fwd_splits(RT, CTv, device_cus_or_default(a->device));
  const int fgrid = 8 * nsplit * ((RT + 7) / 8);
  int maxgrid = std::max(fgrid, std::max(map_tile_grid((int)(P / 256), CTd), map_tile_rr_grid(CTd, CTv)));
  const size_t need = (size_t)maxgrid * 256 * 4 + 2 * 1024 * sizeof(long long);
  if (scratch_bytes < need) return fail(SCE_EINVAL, "scratch too small: %zu < %zu", scratch_bytes, need);
  float* out = (float*)scratch;
  long long* clk = (long long*)((uint8_t*)scratch + (size_t)maxgrid * 256 * 4);
  auto pass = [&]() {
    if (which == SCE_K_FWD) {
      FwdParams p = {};
      p.xq = xq; p.wqt = wqt; p.dp = S.dp; p.ldx = S.ldx; p.Np = (int)S.Np; p.RT = RT; p.CT = CTv; p.S = nsplit;
      floor_fwd_kernel<<<fgrid, NTHREADS, SMEM_BYTES, st>>>(p, out, clk);
    } else if (which == SCE_K_DX) {
      for (int64_t p0 = 0; p0 < S.Np; p0 += P) {
        const int64_t prow = (S.Np - p0 < P) ? (S.Np - p0) : P;
        DxParams p = {};
        p.wq = wq; p.ghat_t = ghat_t + (p0 / 256) * (S.Vp / BK) * BLOCKED_KSTEP; p.gexp = gexp + p0 / BK; p.kbw = S.Np / BK; p.Vp = S.Vp;
        p.RT = (int)(prow / 256); p.CT = CTd;
        floor_dx_kernel<<<map_tile_grid(p.RT, CTd), NTHREADS, smem_scaled((int)(S.Vp / BK), 0), st>>>(p, out, clk);
      }
    } else {
      DwParams p = {};
      p.xt = (const uint8_t*)a->workspace + B.off_xt; p.ghat_t = ghat_t; p.gexp = gexp; p.kbn = S.Np / BK; p.kbw = S.Np / BK; p.kb0 = 0; p.Vp = S.Vp; p.kbv = S.Vp / BK;
      p.RT = CTd; p.CT = CTv; p.KT = (int)(S.Np / BK);
      floor_dw_kernel<<<map_tile_rr_grid(CTd, CTv), NTHREADS, smem_scaled(p.KT, 0), st>>>(p, out, clk);
    }
  };
  EventPair ev;
  HIP_TRY(ev.create());
  pass();      // warm-up
  HIP_TRY(hipEventRecord(ev.e0, st));
  for (int r = 0; r < reps; ++r) pass();
  HIP_TRY(hipEventRecord(ev.e1, st));
  HIP_TRY(hipEventSynchronize(ev.e1));
  HIP_TRY(hipGetLastError());
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, ev.e0, ev.e1));
  std::vector<long long> h(2 * 1024);
  HIP_TRY(hipMemcpy(h.data(), clk, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
  *ms_per_pass = ms / reps;
  *shader_mhz = median_mhz(h.data(), 250);
  return SCE_OK;
}

