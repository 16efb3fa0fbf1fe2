// Shared definitions for the gfx950 loss-head kernels (internal header).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sce {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// One workgroup (4 wavefronts of 64) owns a TM x TN tile of C = A * B^T where both
// operands are stored K-contiguous ("NT").  A rows land on the accumulator registers,
// B rows on the lanes (v_mfma_f32_32x32x64_f8f6f4: lane l holds column l%32 and rows
// 8*(r/4) + 4*(l/32) + r%4, r = 0..15).
constexpr int TM = 256;          // A-side rows per tile
constexpr int TN = 256;          // B-side rows per tile
constexpr int BK = 128;          // K bytes per LDS slot row
constexpr int SLOT_BYTES = (TM + TN) * BK;      // 65536
constexpr int SMEM_BYTES = 2 * SLOT_BYTES;      // 131072 of the 163840 B a workgroup may hold
constexpr int NTHREADS = 256;
constexpr int SMEM_MAX = 160 * 1024;              // LDS a workgroup may hold on gfx950

constexpr float LOG2E = 1.4426950408889634f;
constexpr int LONG_SEG = 16;     // target columns hit by at least this many rows get their own reduction kernel
constexpr int LONG_CHUNK = 256;  // ... which handles at most about this many rows per workgroup

// Lane index within the wavefront, computed from the execution mask each time it is asked for.  Kernels
// that loop over tiles use this (and a wave index kept in a scalar register) instead of threadIdx.x:
// a value derived from threadIdx.x stays live across the main loop, is spilled there, and its reload
// -- a vector memory load -- makes the next wait count include the tile loads already in flight.
__device__ __forceinline__ int lane_id() {
  unsigned all = ~0u;
  asm volatile("" : "+s"(all));      // a value the optimiser cannot see through: every call computes the index anew
  return (int)__builtin_amdgcn_mbcnt_hi(all, __builtin_amdgcn_mbcnt_lo(all, 0u));
}

static inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }
// Row stride of an MFMA operand with K = k bytes (a multiple of 256): the next odd multiple of 128.
// With an even multiple the 256 rows of a tile fall on few L2 channels (measured: up to 9 % slower).
static inline int64_t row_stride(int64_t k) { return k + 128; }

// Layout of the state sce_forward saves for sce_backward (byte offsets into `saved`).  The two
// quantised copies of W come last; with a caller-provided weight cache they live there instead
// (same relative offsets) and `saved` ends at x_total.
struct SavedLayout {
  int64_t ldx;                       // row stride in bytes of the [..][dp] e4m3 arrays
  int64_t N, d, V, Np, dp, dq, Vp;   // all padded sizes are multiples of 256 (every K loop runs over an even number of 128-byte blocks); dp: row bytes of X_q / W_q^T (= dq for e4m3)
  size_t off_hdr, off_xq, off_lse, off_umax, off_zy, off_rstd, off_lam, x_total;
  size_t rel_wqt, rel_wq, w_total;   // relative to the start of the W region
  size_t total;                      // x_total + w_total
  size_t rel_g, rel_gexp, g_total;   // dlogits emitted by the forward pass (optional; behind whatever else `saved` holds)
};
// hdr: int32 n_valid, int32 n_bad_targets, float mean loss, float pad

// eb: bytes per operand element, 1 (e4m3) or 2 (bf16 operands: forward only, so no second copy of W)
static inline SavedLayout saved_layout(int64_t N, int64_t d, int64_t V, int n_predict, int eb = 1) {
  SavedLayout L;
  L.N = N; L.d = d; L.V = V;
  L.Np = round_up(N, 256); L.dp = round_up(d * eb, 256); L.dq = round_up(d, 256); L.Vp = round_up(V, 256);
  L.ldx = row_stride(L.dp);
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t r = o; o += (bytes + 255) / 256 * 256; return r; };
  L.off_hdr = take(256);
  L.off_xq = take((size_t)L.Np * L.ldx);       // X_q   [Np][dp]  e4m3, zero padded, row stride ldx
  L.off_lse = take((size_t)L.Np * 4);
  L.off_umax = take((size_t)L.Np * 4);
  L.off_zy = take((size_t)L.Np * 4 * n_predict);
  L.off_rstd = take((size_t)L.Np * 4);         // 1 / rms of each row when the final norm is part of the call
  L.off_lam = take((size_t)L.Np * 4);          // per-row exponent boost of the dlogits (an integer in a float)
  L.x_total = o;
  o = 0;
  L.rel_wqt = take((size_t)L.Vp * L.ldx);      // W_q^T [Vp][dp], row stride ldx
  L.rel_wq = take(eb == 1 ? (size_t)L.dq * L.Vp : 0);        // W_q: dq rows, K = Vp, tile by tile (256 rows x 128 B per K block)
  L.w_total = o;
  L.total = L.x_total + L.w_total;
  o = 0;
  L.rel_g = take((size_t)L.Vp * L.Np);                          // G, Np rows, K = Vp, tile by tile
  L.rel_gexp = take((size_t)(L.Vp / 128) * (L.Np / 128) * 4);   // its block exponents
  L.g_total = o;
  return L;
}

struct BwdLayout {
  int64_t P, Pw;                     // rows per recompute/dX panel and per dW launch (multiples of 256, Pw of P)
  size_t off_gexp, off_rho, off_rowinfo, off_hcoef, off_blockmax, off_xi, off_xt, off_dwacc, off_perm, off_keys,
      off_segoff, off_longlist, off_longbase, off_longsum, off_sorttmp, off_dxpart, off_ghat_t, fixed, total;
  size_t sorttmp_bytes, part_stride;   // part_stride: bytes between consecutive fp32 dW partials
  size_t off_dwtail, tail_bytes;       // partial tiles of the K-split last round of dW: behind `total`, used when the workspace reaches that far
  int nparts;
};

}  // namespace sce
