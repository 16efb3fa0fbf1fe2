// Backward kernels: row factors, transposed scaled X, recompute, dX, dW (with its K-split last round), the one-hot
// part of dW from the sorted targets, finalisation (internal header).
// Part of the one translation unit sce_kernels.hip, which includes it after the headers it builds on.
#pragma once

namespace sce {

// ------------------------------------------------------------------------------------------
// backward
// ------------------------------------------------------------------------------------------
// per row: rho (row factor of the block-scaled dlogits) and h_k (one-hot coefficients).
//   dz_iv = g_i ( S_i p_iv - sum_k w_k [v = y_{i+k}] ),  S_i = sum of w_k over the offsets that take part,
//   S_i p_iv (1 - t^2) = rho_i (D_iv 2^{lam_i})  with  rho_i = g_i S_i e^{cap - lse_i} 2^{-lam_i}.
// The target columns take no part in D (take_target_logits knocks them out where D is formed): their S_i p_iy goes into the
// one-hot coefficient instead, h_ik = g_i (1 - t_y^2) (w_k - S_i p_iy), formed here in fp32 from lse and z_y.
// Through e4m3 the difference S_i p_iy - w_k would carry the rounding error of p_iy alone, a relative
// error of eps p / (1 - p) that grows without bound on rows the model is sure of.  When two offsets of a row
// have the same target, the first one carries the S_i p_iy term.
__global__ __launch_bounds__(256) void bwd_prep_kernel(const float* __restrict__ s_lse,
                                                      const float* __restrict__ s_zy, const int64_t* __restrict__ targets,
                                                      int64_t ignore_index, const int32_t* __restrict__ hdr,
                                                      const float* __restrict__ grad_output, int per_row, float grad_scale,
                                                      const float* __restrict__ mtp_weights, int n_predict,
                                                      float cap, int N, int Np, int V, const float* __restrict__ lam,
                                                      float* __restrict__ rho, float* __restrict__ hcoef,
                                                      float* __restrict__ blockmax, int32_t* __restrict__ rowinfo, CallMode mode) {
  __shared__ float smax[256];
  const int i = blockIdx.x * 256 + threadIdx.x;
  float r = 0.f;
  float h[4] = {0.f, 0.f, 0.f, 0.f};
  // the forward call that wrote `saved` was asked for something else (kept dlogits, vocabulary limit, offsets, cap):
  // its state does not fit this call, and every gradient comes out NaN rather than silently wrong
  const CallMode fm = *reinterpret_cast<const CallMode*>(reinterpret_cast<const uint8_t*>(hdr) + HDR_MODE_OFF);
  const bool mismatch = fm.emit != mode.emit || fm.vocab_limit != mode.vocab_limit || fm.n_predict != mode.n_predict || fm.cap_bits != mode.cap_bits;
  // The row's exponent boost.  A forward pass that emitted the dlogits had to estimate the row's sum from a sample of
  // the row (fwd_sample_kernel).  When the dlogits are formed again here in backward, the sum Z = e^{lse - cap} is known, and
  // the boost is what makes the stored value the probability itself, D 2^lam = p (1 - t^2): rows
  // that share a block are then weighed by what their entries contribute, whatever the shapes of their distributions.
  float lam_i = 0.f;
  if (i < N) lam_i = rowinfo ? (cap - s_lse[i]) * LOG2E : lam[i];
  if (!(lam_i >= -64.f && lam_i <= 120.f)) lam_i = 0.f;      // (ignored rows have no lse to speak of)
  if (rowinfo && i < Np) {          // what the recompute kernel wants to know of a row: its boost and its target columns
    rowinfo[i] = __float_as_int(lam_i);
    for (int k = 0; k < 4; ++k)
      rowinfo[(int64_t)(1 + k) * Np + i] = (k < n_predict && i < N && target_valid(targets, ignore_index, i + k, N, V)) ? (int)targets[i + k] : -1;
    for (int k = 0; k < 4; ++k)          // and the target logits as the forward pass saved them: the recompute kernel knows its targets by these values
      rowinfo[(int64_t)(5 + k) * Np + i] = (k < n_predict && i < N) ? __float_as_int(s_zy[(int64_t)k * Np + i]) : 0x7fc00000;
  }
  if (i < N) {
    const float g = (per_row ? grad_output[i] : grad_output[0] / (float)hdr[0]) * grad_scale;
    float sw = 0.f;
    bool ok[4] = {false, false, false, false};
    int64_t yk[4] = {0, 0, 0, 0};
    for (int k = 0; k < n_predict; ++k) {
      ok[k] = target_valid(targets, ignore_index, i + k, N, V);
      if (!ok[k]) continue;
      yk[k] = targets[i + k];
      sw += mtp_weights ? mtp_weights[k] : 1.0f;
    }
    if (ok[0] || ok[1] || ok[2] || ok[3]) {
      const float lse = s_lse[i];
      for (int k = 0; k < n_predict; ++k) {
        if (!ok[k]) continue;
        const float wk = mtp_weights ? mtp_weights[k] : 1.0f;
        const float zy = s_zy[(int64_t)k * Np + i];
        const float ty = zy / cap;
        bool first = true;
        for (int k2 = 0; k2 < k; ++k2) first = first && !(ok[k2] && yk[k2] == yk[k]);
        h[k] = g * (1.0f - ty * ty) * (wk - (first ? sw * expf(zy - lse) : 0.f));
      }
      // the stored dlogits carry the row's boost 2^lam: an integer from the forward pass that emitted them, the real
      // (cap - lse) log2(e) here -- then rho_i 2^-lam_i is g_i times the row's weights and nothing else, the same number for
      // nearly every row of a mean-reduced loss, and the scaled X that dW multiplies with is X_q itself: no second rounding
      r = rowinfo ? g * sw * expf(cap - lse - lam_i * 0.6931471805599453f) : ldexpf(g * sw * expf(cap - lse), -(int)lam_i);
    }
  }
  if (mismatch && i < N) {
    r = NAN;
    for (int k = 0; k < 4; ++k) h[k] = NAN;
  }
  if (i < Np) {
    rho[i] = r;
    for (int k = 0; k < n_predict; ++k) hcoef[(int64_t)k * Np + i] = h[k];
  }
  smax[threadIdx.x] = fabsf(r);
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (threadIdx.x < w) smax[threadIdx.x] = fmaxf(smax[threadIdx.x], smax[threadIdx.x + w]);
    __syncthreads();
  }
  if (threadIdx.x == 0) blockmax[blockIdx.x] = smax[0];
}

__global__ __launch_bounds__(1024) void bwd_xi_kernel(const float* __restrict__ blockmax, int n, float* __restrict__ xi) {
  __shared__ float smax[1024];
  float m = 0.f;
  for (int i = threadIdx.x; i < n; i += 1024) m = fmaxf(m, blockmax[i]);
  smax[threadIdx.x] = m;
  __syncthreads();
  for (int w = 512; w > 0; w >>= 1) {
    if (threadIdx.x < w) smax[threadIdx.x] = fmaxf(smax[threadIdx.x], smax[threadIdx.x + w]);
    __syncthreads();
  }
  if (threadIdx.x == 0) xi[0] = (smax[0] > 0.f && isfinite(smax[0])) ? smax[0] : 1.0f;
}

// Xt (blocked, dq rows, K = Np) = e4m3( X_q[i][j] * rho_i / xi ), transposed through LDS in 128 x 128 tiles: a row of
// the tile is one whole 128-byte line of the blocked layout on the way out, and 128 bytes of an X_q row on the way in.
constexpr int XT_TILE = 128;
__global__ __launch_bounds__(256) void bwd_xt_kernel(const uint8_t* __restrict__ xq, int64_t dp, int64_t ldx, int64_t kbn,
                                                    const float* __restrict__ rho, const float* __restrict__ xi,
                                                    uint8_t* __restrict__ xt) {
  __shared__ uint8_t tile[XT_TILE][XT_TILE + 4];
  const int t = threadIdx.x;
  const int64_t i0 = (int64_t)blockIdx.x * XT_TILE, j0 = (int64_t)blockIdx.y * XT_TILE;
  if (j0 < dp) {
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int r = (t >> 3) + 32 * pass, c = (t & 7) * 16;
      const v4i raw = *reinterpret_cast<const v4i*>(xq + (i0 + r) * ldx + j0 + c);
      const float f = rho[i0 + r] / xi[0];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const uint32_t w = (uint32_t)raw[m];
        const uint32_t o = cvt4_e4m3(e4m3_to_float<0>(w) * f, e4m3_to_float<1>(w) * f, e4m3_to_float<2>(w) * f,
                                     e4m3_to_float<3>(w) * f);
        *reinterpret_cast<uint32_t*>(&tile[r][c + 4 * m]) = o;
      }
    }
  } else {
    for (int e = t; e < XT_TILE * (XT_TILE + 4) / 4; e += 256) reinterpret_cast<uint32_t*>(&tile[0][0])[e] = 0;
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int jr = (t >> 3) + 32 * pass, ic = (t & 7) * 16;
    uint32_t out[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      out[m] = (uint32_t)tile[ic + 4 * m][jr] | ((uint32_t)tile[ic + 4 * m + 1][jr] << 8) |
               ((uint32_t)tile[ic + 4 * m + 2][jr] << 16) | ((uint32_t)tile[ic + 4 * m + 3][jr] << 24);
    }
    *reinterpret_cast<v4i*>(xt + blocked_offset(j0 + jr, i0 + ic, kbn)) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
  }
}

struct RecomputeParams {
  const uint8_t* xq;     // [Np][dp], already offset to the panel's first row
  const uint8_t* wqt;    // [Vp][dp]
  uint8_t* ghat_t;       // G of the rows this buffer stands for, tile by tile (kbv blocks of 128 columns per tile of 256 rows)
  uint32_t* gexp;        // [Vp / 128][kbw]
  const int32_t* rowinfo;      // [ROWINFO_PLANES][Np], offset to the panel's first row: boosts and targets (bwd_prep_kernel)
  int64_t Np;
  int n_predict;
  int64_t dp, ldx;             // K extent and row stride of xq / wqt
  int64_t kbw, kb0, kbv;       // blocks of 128 rows in the buffer (row stride of gexp), block of this panel's first row, blocks of 128 columns
  int RT, CT, V;
  float k1, c2, sc;      // as in FwdParams
  const DevConsts* dc;   // non-NULL: k1 and sc come from here
};

// Recompute a 256 x 256 logit tile and leave its block-scaled dlogits in G (16-byte stores straight from the registers).
constexpr int ROWINFO_PLANES = 9;                      // per row: exponent boost (a float), the target column of each of 4 offsets (or -1), the target logits
constexpr int SMEM_RECOMPUTE = SMEM_BYTES + 4 * ROWINFO_PLANES * 512;      // two K slots + the row data of 128 rows per wave

__global__ __launch_bounds__(256) void bwd_recompute_kernel(RecomputeParams p_in) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  RecomputeParams p = p_in;
  if (p.dc) { p.k1 = p.dc->k1; p.sc = p.dc->sc; }
  int rt, ct;
  if (!map_tile(blockIdx.x, p.RT, p.CT, rt, ct)) return;
  // The tile order goes through the columns in groups of 8, and it does so from the last group to the first:
  // the dX kernel that follows starts its K loop at column 0, with the part of G that was written last and is
  // still in the memory-side cache.
  ct = p.CT - 1 - ct;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wa = wave >> 1, wb = wave & 1;
  // The boosts and targets of the wave's 128 rows go straight to LDS, behind the two slots: requested before the K
  // loop (whose waits for its own, younger loads cover them), read after it, no register held in between.
  // (Through the compiler's builtin, which knows that the instruction reads M0 and sets it itself; the price -- the
  // compiler makes the first LDS read after it wait for every vector memory load in flight, the tile loads of the
  // main loop's prologue included -- is paid once per tile here.)
  {
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    typedef const __attribute__((address_space(1))) int32_t global_i32;
    lds_u8* dst = (lds_u8*)(smem + SMEM_BYTES) + wave * (ROWINFO_PLANES * 512);
    const int lane = lane_id();
#pragma unroll
    for (int q = 0; q < ROWINFO_PLANES; ++q) {
      global_i32* src = (global_i32*)(uintptr_t)(p.rowinfo + (int64_t)q * p.Np + rt * 256 + wb * 128 + lane);
      // lane l's dword lands at the LDS base + 4 l; the instruction's offset moves the memory address and the LDS
      // address alike: the second half of the rows
      __builtin_amdgcn_global_load_lds(src, dst + q * 512, 4, 0, 0);
      __builtin_amdgcn_global_load_lds(src, dst + q * 512, 4, 256, 0);
    }
  }
  v16f acc[4][4];
  // (as in the forward kernel: the last pair's MFMAs of row blocks 1 - 3 ride along with the epilogues of row blocks 0 and 1)
  mfma_mainloop<false, NoHook, BK, false, 0, false, true>(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, p.xq + (int64_t)rt * 256 * p.ldx, p.ldx, (int)(p.dp / BK), smem, acc, 2 * (rt & 3), ct & 7, wave);
  DeferredTail deferred(smem, wa, wb);
  auto tail = [&](int b, int k) { deferred(acc, b, k); };
  const int vlim = p.V - ct * 256;           // columns >= vlim of this tile do not exist
  const bool ragged = vlim < 256;
  const float* lam = reinterpret_cast<const float*>(smem + SMEM_BYTES) + wave * (ROWINFO_PLANES * 128);     // row block b: 32 floats on
  const int* tgt = reinterpret_cast<const int*>(smem + SMEM_BYTES) + wave * (ROWINFO_PLANES * 128) + 128;
  uint8_t* gq = const_cast<uint8_t*>(uniform_ptr(p.ghat_t + ((p.kb0 / 2 + rt) * p.kbv + 2 * ct + wa) * BLOCKED_KSTEP + wb * 128 * BK));      // the wave's quadrant of G
  const int col0 = ct * 256 + wa * 128;
  // The target entries are not looked up in the accumulators (the compiler moves a row block's 64 accumulators around
  // every such lookup): a lane knows the value of a target among its columns -- the forward pass saved it, and this
  // kernel computes the same number -- and keeps it out of the block exponent by that (form_dlogits, EXCL); the bytes
  // are cleared afterwards (fwd_knock_kernel).
  const float* tval = reinterpret_cast<const float*>(tgt + 4 * 128);
  auto target_value = [&](int b) {
    float v = __builtin_nanf("");
    for (int k = 0; k < p.n_predict; ++k) {
      const int rel = tgt[k * 128 + b * 32 + (lane_id() & 31)] - col0;
      if ((unsigned)rel < 128u && ((rel >> 2) & 1) == (lane_id() >> 5)) v = tval[k * 128 + b * 32 + (lane_id() & 31)];
    }
    return v;
  };
  float xc[4];
  if (ragged) strike_columns_beyond<0, 1>(acc, vlim, wa);
  xc[0] = target_value(0);
  uint32_t ew = form_dlogits<false, 32, 32, 0, 1, decltype(tail)&, true>(acc, p.k1, p.c2, 0, gq, wa, wb, nullptr, lam, false, tail, xc, p.sc);
  if (ragged) strike_columns_beyond<1, 2>(acc, vlim, wa);
  xc[1] = target_value(1);
  ew |= form_dlogits<false, 32, 32, 1, 2, decltype(tail)&, true>(acc, p.k1, p.c2, 0, gq, wa, wb, nullptr, lam, false, tail, xc, p.sc);
  if (ragged) strike_columns_beyond<2, 4>(acc, vlim, wa);
  xc[2] = target_value(2); xc[3] = target_value(3);
  NoHook none;
  ew |= form_dlogits<false, 32, 32, 2, 4, NoHook&, true>(acc, p.k1, p.c2, 0, gq, wa, wb, nullptr, lam, false, none, xc, p.sc);
  if (lane_id() == 0) p.gexp[(int64_t)(2 * ct + wa) * p.kbw + p.kb0 + 2 * rt + wb] = ew;
}

struct DxParams {
  const uint8_t* wq;      // dq rows, K = Vp, tile by tile: A side (rows j)
  const uint8_t* ghat_t;  // G, tile by tile (rows i, K = v); already at the tile of the panel's first row    B side (rows i of the panel)
  const uint32_t* gexp;   // its block exponents [Vp / 128][kbw], likewise at the panel's first row
  const uint8_t* wqt;     // [Vp][dp]   for the one-hot gather
  const float* rho;       // offset to the panel
  const float* hcoef;     // [n_predict][Np], offset to the panel
  const int64_t* targets; // offset to the panel
  void* dx;               // offset to the panel's first row
  float* part;            // [ksplit][RT * 256][dq] fp32 partial sums (ksplit > 1 only)
  int64_t dx_ld, Vp, ldx, Np, dq;        // Vp: K extent; ldx: row stride of wqt
  int64_t kbw;                           // blocks of 128 rows i that gexp counts per block of 128 columns
  int RT, CT, rows, d, V;  // rows: valid rows in this panel
  int n_predict, rows_left; // rows_left: N - (first row of the panel), bounds the target look-ahead
  int ksplit;              // the K loop (V) is cut into this many parts, one workgroup each
  float w_s;
  const DevConsts* dc;     // non-NULL: w_s comes from here
};

// LDS a wave uses to stage its quadrant of a dX tile on the way out: 128 rows of 64 fp32 (or bf16) plus 16 bytes
constexpr int DX_STAGE_BYTES = 128 * (64 * 4 + 16);
constexpr int SMEM_DX = 4 * DX_STAGE_BYTES > SMEM_BYTES ? 4 * DX_STAGE_BYTES : SMEM_BYTES;
// ... or the two K slots and, behind them, the block exponents of the K loop (one dword per K block and half of the rows)
constexpr int MAX_SCALE_KBLOCKS = (SMEM_MAX - SMEM_BYTES) / 8;      // K blocks of one scaled main loop: 4096
static inline int smem_scaled(int kblocks, int at_least) { const int n = SMEM_BYTES + 8 * kblocks; return n > at_least ? n : at_least; }

// Row scale and one-hot term of four consecutive dX columns j..j+3 of panel row il:
//   dX = rho_i w_s (G W_q^T) - sum_k h_ik w_s W_q^T[y_{i+k}, :]
struct DxRowTerms {
  float rs;
  float hs[4];
  const uint8_t* wrow[4];
  __device__ __forceinline__ DxRowTerms(const DxParams& p, int il) {
    rs = p.rho[il] * p.w_s;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      hs[k] = 0.f; wrow[k] = p.wqt;
      if (k < p.n_predict && il + k < p.rows_left) {
        const float hk = p.hcoef[(int64_t)k * p.Np + il] * p.w_s;
        const int64_t y = p.targets[il + k];
        if (hk != 0.f && y >= 0 && y < p.V) { hs[k] = hk; wrow[k] = p.wqt + y * p.ldx; }
      }
    }
  }
  template <typename T>
  __device__ __forceinline__ void store4(const DxParams& p, T* dst, int j, float o0, float o1, float o2, float o3) const {
    // explicit roundings: the fast path of bwd_dx_kernel forms the same values and must give the same bits
    o0 = __fmul_rn(o0, rs); o1 = __fmul_rn(o1, rs); o2 = __fmul_rn(o2, rs); o3 = __fmul_rn(o3, rs);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (k < p.n_predict) {
        const uint32_t w = *reinterpret_cast<const uint32_t*>(wrow[k] + j);
        o0 = __builtin_fmaf(-hs[k], e4m3_to_float<0>(w), o0); o1 = __builtin_fmaf(-hs[k], e4m3_to_float<1>(w), o1);
        o2 = __builtin_fmaf(-hs[k], e4m3_to_float<2>(w), o2); o3 = __builtin_fmaf(-hs[k], e4m3_to_float<3>(w), o3);
      }
    }
    Elem<T>::store(dst + 0, o0); Elem<T>::store(dst + 1, o1);
    Elem<T>::store(dst + 2, o2); Elem<T>::store(dst + 3, o3);
  }
};

// SPLIT = false: one workgroup per 256 x 256 tile of dX, whole K loop, finished values stored.
// SPLIT = true : a panel with too few tiles to fill the chip; each tile's K loop is shared by ksplit
//                workgroups that store raw fp32 partial sums, and bwd_dx_finish_kernel adds them up.
template <typename T, bool SPLIT>
__global__ __launch_bounds__(256) void bwd_dx_kernel(DxParams p_in) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  DxParams p = p_in;
  if (p.dc) p.w_s = p.dc->w_s;
  int rt, ct, ks = 0;
  if (!map_tile(blockIdx.x, p.RT, SPLIT ? p.CT * p.ksplit : p.CT, rt, ct)) return;
  int64_t k0 = 0;
  int KD = (int)(p.Vp / BK);
  if (SPLIT) {
    ks = ct % p.ksplit; ct /= p.ksplit;
    const int pairs = KD >> 1;
    const int q0 = (int)((int64_t)pairs * ks / p.ksplit), q1 = (int)((int64_t)pairs * (ks + 1) / p.ksplit);
    k0 = (int64_t)q0 * 2 * BK; KD = 2 * (q1 - q0);
  }
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wa = wave >> 1, wb = wave & 1;
  // the block exponents of this tile's K loop wait in LDS behind the two K slots: [i half][K block]
  uint32_t* lsc = reinterpret_cast<uint32_t*>(smem + SMEM_BYTES);
  for (int e = t; e < 2 * KD; e += NTHREADS) {
    const int w = e >= KD, kb = e - w * KD;
    lsc[e] = p.gexp[(k0 / BK + kb) * p.kbw + 2 * rt + w];
  }
  __syncthreads();
  v16f acc[4][4];
  // both operands tile by tile with K = v: W_q rows j, G rows i
  mfma_mainloop<false, NoHook, BLOCKED_KSTEP, false, 1>(p.wq + ((int64_t)ct * (p.Vp / BK) + k0 / BK) * BLOCKED_KSTEP, BK,
                                                        p.ghat_t + ((int64_t)rt * (p.Vp / BK) + k0 / BK) * BLOCKED_KSTEP, BK, KD, smem, acc,
                                                        2 * (rt & 3), ct & 7, __builtin_amdgcn_readfirstlane(wave), NoHook(), 0, 0,
                                                        lsc + __builtin_amdgcn_readfirstlane(wb) * KD);
  const int jbase = ct * 256 + wa * 128 + 4 * (lane >> 5);
  T* dx = reinterpret_cast<T*>(p.dx);
  if (!SPLIT && p.n_predict > 1 && ((reinterpret_cast<uintptr_t>(p.dx) | (uintptr_t)(p.dx_ld * (int64_t)sizeof(T))) & 15) == 0) {
    // Several prediction offsets: the same staged way out as below, with the W_q^T words of all offsets loaded for one
    // block of 32 rows and 64 columns at a time (all at once they would not fit the registers; folded into the
    // accumulators beforehand, offset by offset, the whole kernel, main loop included, takes to scratch memory).
    // Values and their order are those of DxRowTerms::store4.
    const int K = p.n_predict;
    float rs[4], hs[4][4];
    int yrow[4][4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int il = rt * 256 + wb * 128 + b * 32 + (lane & 31);
      const bool live = il < p.rows;
      rs[b] = p.rho[live ? il : 0] * p.w_s;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        hs[b][k] = 0.f; yrow[b][k] = 0;
        if (k < K) {
          const bool there = live && il + k < p.rows_left;
          const float hk = there ? p.hcoef[(int64_t)k * p.Np + il] * p.w_s : 0.f;
          const int64_t y = there ? p.targets[il + k] : -1;
          if (hk != 0.f && y >= 0 && y < p.V) { hs[b][k] = hk; yrow[b][k] = (int)y; }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    constexpr int RB = 64 * (int)sizeof(T), PITCH = RB + 16, CH = RB / 16;     // row bytes, staging pitch, chunks per row
    uint8_t* stg = smem + wave * DX_STAGE_BYTES;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        uint32_t wk[4][8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (k < K) {
            const uint8_t* wrow = p.wqt + (int64_t)yrow[b][k] * p.ldx + jbase + pass * 64;
#pragma unroll
            for (int e = 0; e < 8; ++e) wk[k][e] = *reinterpret_cast<const uint32_t*>(wrow + (e >> 2) * 32 + 8 * (e & 3));
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        uint8_t* srow = stg + (b * 32 + (lane & 31)) * PITCH + 4 * (lane >> 5) * (int)sizeof(T);
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int a = 2 * pass + a2;
            float o0 = __fmul_rn(acc[a][b][4 * q + 0], rs[b]), o1 = __fmul_rn(acc[a][b][4 * q + 1], rs[b]);
            float o2 = __fmul_rn(acc[a][b][4 * q + 2], rs[b]), o3 = __fmul_rn(acc[a][b][4 * q + 3], rs[b]);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              if (k < K) {
                const uint32_t w = wk[k][a2 * 4 + q];
                o0 = __builtin_fmaf(-hs[b][k], e4m3_to_float<0>(w), o0); o1 = __builtin_fmaf(-hs[b][k], e4m3_to_float<1>(w), o1);
                o2 = __builtin_fmaf(-hs[b][k], e4m3_to_float<2>(w), o2); o3 = __builtin_fmaf(-hs[b][k], e4m3_to_float<3>(w), o3);
              }
            }
            uint8_t* dst = srow + (a2 * 32 + 8 * q) * (int)sizeof(T);
            if constexpr (sizeof(T) == 2)
              *reinterpret_cast<v2i*>(dst) = (v2i){(int)((uint32_t)float_to_bf16_bits(o0) | ((uint32_t)float_to_bf16_bits(o1) << 16)),
                                                   (int)((uint32_t)float_to_bf16_bits(o2) | ((uint32_t)float_to_bf16_bits(o3) << 16))};
            else
              *reinterpret_cast<v4f*>(dst) = (v4f){o0, o1, o2, o3};
          }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int n = 0; n < 128 * CH / 64; ++n) {
        const int c = lane + 64 * n, row = c / CH, k16 = c % CH;
        const int il = rt * 256 + wb * 128 + row;
        const int col = ct * 256 + wa * 128 + pass * 64 + k16 * (16 / (int)sizeof(T));
        if (il < p.rows && col < p.d)
          *reinterpret_cast<v4i*>(reinterpret_cast<uint8_t*>(dx) + ((int64_t)il * p.dx_ld + col) * (int64_t)sizeof(T)) =
              *reinterpret_cast<const v4i*>(stg + row * PITCH + k16 * 16);
      }
    }
    return;
  }
  if (!SPLIT && p.n_predict == 1) {
    // One wave per SIMD has nothing to hide a load behind, so the epilogue is written in three phases with all
    // loads of a phase in flight together: the row terms of the lane's four rows, then the 64 words of the four
    // W_q^T rows of their targets, then arithmetic and stores.
    float rs[4], hs[4];
    int64_t yy[4];
    int il4[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int il = rt * 256 + wb * 128 + b * 32 + (lane & 31);
      const bool live = il < p.rows;
      il4[b] = live ? il : -1;
      const int is = live ? il : 0;                       // row 0 exists whenever any row does
      rs[b] = p.rho[is] * p.w_s;
      hs[b] = p.hcoef[is] * p.w_s;
      yy[b] = p.targets[is];
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t wv[4][16];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const bool hit = il4[b] >= 0 && hs[b] != 0.f && yy[b] >= 0 && yy[b] < p.V;
      if (!hit) hs[b] = 0.f;
      const uint8_t* wrow = p.wqt + (hit ? yy[b] : 0) * p.ldx + jbase;
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int q = 0; q < 4; ++q) wv[b][4 * a + q] = *reinterpret_cast<const uint32_t*>(wrow + a * 32 + 8 * q);
    }
    __builtin_amdgcn_sched_barrier(0);
    // Out through LDS (free now: every wave is past the closing barrier of the main loop), so that the stores are
    // whole 16-byte runs of a row instead of 8-byte pieces of 32 different rows: each wave stages its own quadrant,
    // 64 columns at a time, and reads only what it wrote itself (no barrier).
    const bool vec = ((reinterpret_cast<uintptr_t>(p.dx) | (uintptr_t)(p.dx_ld * (int64_t)sizeof(T))) & 15) == 0;
    if (vec) {
      constexpr int RB = 64 * (int)sizeof(T), PITCH = RB + 16, CH = RB / 16;     // row bytes, staging pitch, chunks per row
      uint8_t* stg = smem + wave * DX_STAGE_BYTES;
#pragma unroll
      for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          uint8_t* srow = stg + (b * 32 + (lane & 31)) * PITCH + 4 * (lane >> 5) * (int)sizeof(T);
#pragma unroll
          for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int a = 2 * pass + a2;
              const uint32_t w = wv[b][4 * a + q];
              const float o0 = __builtin_fmaf(-hs[b], e4m3_to_float<0>(w), __fmul_rn(acc[a][b][4 * q + 0], rs[b]));
              const float o1 = __builtin_fmaf(-hs[b], e4m3_to_float<1>(w), __fmul_rn(acc[a][b][4 * q + 1], rs[b]));
              const float o2 = __builtin_fmaf(-hs[b], e4m3_to_float<2>(w), __fmul_rn(acc[a][b][4 * q + 2], rs[b]));
              const float o3 = __builtin_fmaf(-hs[b], e4m3_to_float<3>(w), __fmul_rn(acc[a][b][4 * q + 3], rs[b]));
              uint8_t* dst = srow + (a2 * 32 + 8 * q) * (int)sizeof(T);
              if constexpr (sizeof(T) == 2)
                *reinterpret_cast<v2i*>(dst) = (v2i){(int)((uint32_t)float_to_bf16_bits(o0) | ((uint32_t)float_to_bf16_bits(o1) << 16)),
                                                     (int)((uint32_t)float_to_bf16_bits(o2) | ((uint32_t)float_to_bf16_bits(o3) << 16))};
              else
                *reinterpret_cast<v4f*>(dst) = (v4f){o0, o1, o2, o3};
            }
        }
#pragma unroll
        for (int n = 0; n < 128 * CH / 64; ++n) {
          const int c = lane + 64 * n, row = c / CH, k16 = c % CH;
          const int il = rt * 256 + wb * 128 + row;
          const int col = ct * 256 + wa * 128 + pass * 64 + k16 * (16 / (int)sizeof(T));
          if (il < p.rows && col < p.d)
            *reinterpret_cast<v4i*>(reinterpret_cast<uint8_t*>(dx) + ((int64_t)il * p.dx_ld + col) * (int64_t)sizeof(T)) =
                *reinterpret_cast<const v4i*>(stg + row * PITCH + k16 * 16);
        }
      }
      return;
    }
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      if (il4[b] < 0) continue;
      T* drow = dx + (int64_t)il4[b] * p.dx_ld;
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int j = jbase + a * 32 + 8 * q;
          if (j >= p.d) continue;                       // d is a multiple of 4, so j..j+3 are in range together
          const uint32_t w = wv[b][4 * a + q];
          Elem<T>::store(drow + j + 0, __builtin_fmaf(-hs[b], e4m3_to_float<0>(w), __fmul_rn(acc[a][b][4 * q + 0], rs[b])));
          Elem<T>::store(drow + j + 1, __builtin_fmaf(-hs[b], e4m3_to_float<1>(w), __fmul_rn(acc[a][b][4 * q + 1], rs[b])));
          Elem<T>::store(drow + j + 2, __builtin_fmaf(-hs[b], e4m3_to_float<2>(w), __fmul_rn(acc[a][b][4 * q + 2], rs[b])));
          Elem<T>::store(drow + j + 3, __builtin_fmaf(-hs[b], e4m3_to_float<3>(w), __fmul_rn(acc[a][b][4 * q + 3], rs[b])));
        }
    }
    return;
  }
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int il = rt * 256 + wb * 128 + b * 32 + (lane & 31);
    if (SPLIT) {
      float* dst = p.part + ((int64_t)ks * p.RT * 256 + il) * p.dq;
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<v4f*>(dst + jbase + a * 32 + 8 * q) =
              (v4f){acc[a][b][4 * q + 0], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]};
      continue;
    }
    if (il >= p.rows) continue;
    const DxRowTerms row(p, il);
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int j = jbase + a * 32 + 8 * q;
        if (j >= p.d) continue;                       // d is a multiple of 4, so j..j+3 are in range together
        row.store4<T>(p, dx + (int64_t)il * p.dx_ld + j, j, acc[a][b][4 * q + 0], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2],
                      acc[a][b][4 * q + 3]);
      }
    }
  }
}

// sum of the K-split partials, row scale, one-hot term, cast: a thread per (row, four columns)
template <typename T>
__global__ __launch_bounds__(256) void bwd_dx_finish_kernel(DxParams p_in) {
  DxParams p = p_in;
  if (p.dc) p.w_s = p.dc->w_s;
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int per_row = p.d / 4;
  const int il = (int)(q / per_row), j = (int)(q - (int64_t)il * per_row) * 4;
  if (il >= p.rows) return;
  v4f sum = (v4f){0.f, 0.f, 0.f, 0.f};
  for (int ks = 0; ks < p.ksplit; ++ks)      // fixed order
    sum += *reinterpret_cast<const v4f*>(p.part + ((int64_t)ks * p.RT * 256 + il) * p.dq + j);
  const DxRowTerms row(p, il);
  row.store4<T>(p, reinterpret_cast<T*>(p.dx) + (int64_t)il * p.dx_ld + j, j, sum[0], sum[1], sum[2], sum[3]);
}

struct DwParams {
  const uint8_t* xt;      // dq rows, K = Np, blocked                             A side (rows j)
  const uint8_t* ghat_t;  // G, tile by tile (rows i, K = v), already at the tile of this launch's first row      B side (rows v, through the transposing read)
  const uint32_t* gexp;   // its block exponents [Vp / 128][kbw], likewise
  float* dwacc;           // [dq][Vp] fp32
  int64_t kbn, kbw, kb0, Vp;   // K blocks per tile of xt; blocks of 128 rows that gexp counts; first K block of xt in this launch; row length of dwacc
  int64_t kbv;                 // blocks of 128 columns per tile of 256 rows of G
  int RT, CT, KT;
};

// ACC: add to what the partial holds (only when there are more dW launches than partial buffers)
template <bool ACC>
__global__ __launch_bounds__(256) void bwd_dw_kernel(DwParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int rt, ct;
  if (!map_tile_rr(blockIdx.x, p.RT, p.CT, rt, ct)) return;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wa = wave >> 1, wb = wave & 1;
  // the block exponents of this tile's K loop wait in LDS behind the two K slots: [v half][K block]
  uint32_t* lsc = reinterpret_cast<uint32_t*>(smem + SMEM_BYTES);
  for (int e = t; e < 2 * p.KT; e += NTHREADS) {
    const int w = e >= p.KT, kb = e - w * p.KT;
    lsc[e] = p.gexp[(int64_t)(2 * ct + w) * p.kbw + kb];
  }
  __syncthreads();
  v16f acc[4][4];
  // B = G with K (rows i) as the slow index: the 128 rows of a K block are half a tile of G, the 256 columns of this dW
  // tile its column blocks 2 ct and 2 ct + 1 (BLOCKED_KSTEP apart); from one tile of G to the next kbv blocks
  mfma_mainloop<false, NoHook, BLOCKED_KSTEP, true, 2>(p.xt + ((int64_t)rt * p.kbn + p.kb0) * BLOCKED_KSTEP, BK, p.ghat_t + (int64_t)(2 * ct) * BLOCKED_KSTEP, BLOCKED_KSTEP, p.KT,
                                                       smem, acc, ct & 7, 2 * (rt & 3), __builtin_amdgcn_readfirstlane(wave), NoHook(), 128 * BK, p.kbv * BLOCKED_KSTEP,
                                                       lsc + __builtin_amdgcn_readfirstlane(wb) * p.KT);
  const int jbase = rt * 256 + wa * 128 + 4 * (lane >> 5);
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int v = ct * 256 + wb * 128 + b * 32 + (lane & 31);
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = jbase + a * 32 + 8 * (r >> 2) + (r & 3);
        float* dst = p.dwacc + (int64_t)j * p.Vp + v;
        *dst = ACC ? (*dst + acc[a][b][r]) : acc[a][b][r];
      }
    }
  }
}

// The tiles of the last, partly filled round of dW (tile0 .. tile0 + ntail - 1 of the round-robin order), shared out
// along K: a tile's K loop is kp pairs of K blocks long, all of them together W = ntail * kp pairs, and workgroup g takes
// pairs [g share, (g + 1) share) of that line -- the end of one tile and the beginning of the next, when its range
// straddles them.  Piece (g, t) of tile t goes to buf[g + t] as plain stores (g + t grows by one from each piece to the
// next along the line, so no two pieces meet); bwd_dw_final_kernel adds up a tile's pieces in the order of g.
struct DwTail {
  float* buf;
  int tile0, ntail, kp, share;      // tile0 < 0: no tail (every tile is in the fp32 partial)
};
// (grid: workgroups x 2.  A workgroup's range is at most half a tile's K loop long, so it lies in one tile or straddles
// two: blockIdx.y = 0 takes the part in the first tile, blockIdx.y = 1 the part in the second, if there is one.  One piece
// per workgroup, with no loop around the main loop: looping over the pieces, the compiler spilled the accumulators.)
__global__ __launch_bounds__(256) void bwd_dw_tail_kernel(DwParams p, DwTail tl) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int g = blockIdx.x;
  const int pos0 = g * tl.share, end = min(tl.ntail * tl.kp, pos0 + tl.share);
  if (pos0 >= end) return;
  int tt = pos0 / tl.kp, pos = pos0;
  if (blockIdx.y == 1) {
    ++tt; pos = tt * tl.kp;
    if (pos >= end) return;
  }
  // (everything here is uniform, but the divisions leave their results in vector registers: the main loop wants
  // its addresses in scalar ones)
  tt = __builtin_amdgcn_readfirstlane(tt);
  const int k0 = __builtin_amdgcn_readfirstlane(pos - tt * tl.kp), k1 = min(tl.kp, k0 + (end - pos)), KD = __builtin_amdgcn_readfirstlane(2 * (k1 - k0));
  int rt, ct;
  tile_from_index(tl.tile0 + tt, p.RT, p.CT, rt, ct);
  rt = __builtin_amdgcn_readfirstlane(rt); ct = __builtin_amdgcn_readfirstlane(ct);
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wa = wave >> 1, wb = wave & 1;
  uint32_t* lsc = reinterpret_cast<uint32_t*>(smem + SMEM_BYTES);
  for (int e = t; e < 2 * KD; e += NTHREADS) {
    const int w = e >= KD, kb = e - w * KD;
    lsc[e] = p.gexp[(int64_t)(2 * ct + w) * p.kbw + 2 * k0 + kb];
  }
  __syncthreads();
  v16f acc[4][4];
  mfma_mainloop<false, NoHook, BLOCKED_KSTEP, true, 2>(uniform_ptr(p.xt + ((int64_t)rt * p.kbn + p.kb0 + 2 * k0) * BLOCKED_KSTEP), BK,
                                                       uniform_ptr(p.ghat_t + ((int64_t)k0 * p.kbv + 2 * ct) * BLOCKED_KSTEP), BLOCKED_KSTEP,
                                                       KD, smem, acc, ct & 7, 2 * (rt & 3), __builtin_amdgcn_readfirstlane(wave), NoHook(), 128 * BK, p.kbv * BLOCKED_KSTEP,
                                                       lsc + __builtin_amdgcn_readfirstlane(wb) * KD);
  float* dst0 = tl.buf + (size_t)(g + tt) * 65536 + (wa * 128 + 4 * (lane >> 5)) * 256 + wb * 128 + (lane & 31);
#pragma unroll
  for (int b = 0; b < 4; ++b)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) dst0[(a * 32 + 8 * (r >> 2) + (r & 3)) * 256 + b * 32] = acc[a][b][r];
}

// sort keys: one entry per (offset k, row i): key = target y_{i+k} (V if the pair takes no part; targets at or
// beyond the vocabulary limit Vl take no part),
// value = entry id k * Np + i
__global__ __launch_bounds__(256) void bwd_keys_kernel(const int64_t* __restrict__ targets, int64_t ignore_index, int N, int Np, int Vl,
                                                      int V, int n_predict, int32_t* __restrict__ keys, int32_t* __restrict__ vals,
                                                      int32_t* __restrict__ longlist) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e == 0) longlist[0] = 0;        // counter of the long-column list, filled later on the same stream
  if (e >= N * n_predict) return;
  const int k = e / N, i = e - k * N;
  keys[e] = target_valid(targets, ignore_index, i + k, N, Vl) ? (int32_t)targets[i + k] : V;
  vals[e] = k * Np + i;
}

// segoff[v] = first sorted position whose key >= v, v = 0..V+1
__global__ __launch_bounds__(256) void bwd_segoff_kernel(const int32_t* __restrict__ skeys, int N, int V,
                                                        int32_t* __restrict__ segoff) {
  const int pos = blockIdx.x * 256 + threadIdx.x;
  if (pos > N) return;
  const int k = (pos < N) ? skeys[pos] : V + 1;
  const int kprev = (pos > 0) ? skeys[pos - 1] : -1;
  for (int v = kprev + 1; v <= k; ++v) segoff[v] = pos;
}


// A column that is the target of at least LONG_SEG rows has its segment of the sorted list cut into
// nch = ceil(L / LONG_CHUNK) equal chunks (the last one may be shorter); chunk c starts at sorted
// position s0 + c * ceil(L / nch).
__device__ __forceinline__ void long_chunks(int L, int& nch, int& len) {
  nch = (L + LONG_CHUNK - 1) / LONG_CHUNK;
  len = (L + nch - 1) / nch;
}

// List of (column, chunk) pairs of the long columns (order irrelevant: each pair is handled on its
// own).  longlist[0] is the count, then two ints per pair; the position of a pair in the list is the slot of its
// chunk sum, and longbase[v] is the position of column v's first pair.
__global__ __launch_bounds__(256) void bwd_longlist_kernel(const int32_t* __restrict__ segoff, int V, int32_t* __restrict__ longlist,
                                                          int32_t* __restrict__ longbase) {
  const int v = blockIdx.x * 256 + threadIdx.x;
  if (v >= V) return;
  const int L = segoff[v + 1] - segoff[v];
  if (L < LONG_SEG) return;
  int nch, len;
  long_chunks(L, nch, len);
  const int at = atomicAdd(&longlist[0], nch);
  longbase[v] = at;
  for (int c = 0; c < nch; ++c) { longlist[1 + 2 * (at + c)] = v; longlist[2 + 2 * (at + c)] = c; }
}

// One-hot part of dW for the long columns: longsum[slot][:] = sum over the chunk's rows of h_i X_q[i, :].
// One workgroup per (chunk, block of 256 rows of dW); the rows of the chunk are split over 16
// row-lanes (8 independent loads in flight each) and folded in a fixed order, so the result does
// not depend on scheduling.
__global__ __launch_bounds__(256) void bwd_dw_long_kernel(const int32_t* __restrict__ longlist, const int32_t* __restrict__ segoff,
                                                         const int32_t* __restrict__ perm, const float* __restrict__ hcoef,
                                                         const uint8_t* __restrict__ xq, int64_t dp, int64_t ldx, int64_t dq, int Np,
                                                         float* __restrict__ longsum) {
  __shared__ float red[16][256];
  if ((int)blockIdx.x >= longlist[0]) return;
  const int v = longlist[1 + 2 * blockIdx.x], ch = longlist[2 + 2 * blockIdx.x];
  int nch, len;
  long_chunks(segoff[v + 1] - segoff[v], nch, len);
  const int s0 = segoff[v] + ch * len;
  const int L = (segoff[v + 1] - s0) < len ? (segoff[v + 1] - s0) : len;
  const int t = threadIdx.x, c = t & 15, rl = t >> 4;
  const int64_t jb = (int64_t)blockIdx.y * 256;
  float a[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) a[m] = 0.f;
  if (jb + c * 16 < dp) {
    const uint8_t* xcol = xq + jb + c * 16;
    for (int n0 = rl; n0 < L; n0 += 16 * 8) {
      v4i raw[8];
      float h[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int n = n0 + 16 * u;
        const int e = n < L ? perm[s0 + n] : -1;          // entry id k * Np + i
        h[u] = e >= 0 ? hcoef[e] : 0.f;
        raw[u] = *reinterpret_cast<const v4i*>(xcol + (int64_t)(e >= 0 ? e % Np : 0) * ldx);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {        // rows in ascending order within a row-lane
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const uint32_t w = (uint32_t)raw[u][m];
          a[4 * m + 0] = fmaf(h[u], e4m3_to_float<0>(w), a[4 * m + 0]);
          a[4 * m + 1] = fmaf(h[u], e4m3_to_float<1>(w), a[4 * m + 1]);
          a[4 * m + 2] = fmaf(h[u], e4m3_to_float<2>(w), a[4 * m + 2]);
          a[4 * m + 3] = fmaf(h[u], e4m3_to_float<3>(w), a[4 * m + 3]);
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < 16; ++m) red[rl][c * 16 + m] = a[m];
  __syncthreads();
  float sfold = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k) sfold += red[k][t];
  longsum[(int64_t)blockIdx.x * dq + jb + t] = sfold;
}

// dW = x_s * ( xi * (sum of the dW partials) - sum over the target segment of h_i X_q[i, :] ), cast to the output
// type; the segment sum is formed here for short segments and read from the chunk sums for long ones.  A thread
// owns one column v and 16 consecutive rows j.
template <typename T>
__global__ __launch_bounds__(256) void bwd_dw_final_kernel(const float* __restrict__ dwacc, int nparts, int64_t part_stride, int64_t Vp, const int32_t* __restrict__ segoff,
                                                          const int32_t* __restrict__ perm, const float* __restrict__ hcoef,
                                                          const uint8_t* __restrict__ xq, int64_t ldx, int Np, const float* __restrict__ xi,
                                                          const float* __restrict__ longsum, const int32_t* __restrict__ longbase, int64_t dq,
                                                          float x_s_host, const DevConsts* __restrict__ dc, int d, int V, T* __restrict__ dw, int64_t dw_ld,
                                                          DwTail tl, int RT, int CT) {
  const float x_s = dc ? dc->x_s : x_s_host;
  const int t = threadIdx.x;
  const int v = blockIdx.x * 64 + (t & 63);
  const int j0 = blockIdx.y * 64 + (t >> 6) * 16;
  if (v >= V || j0 >= d) return;
  const float scale = x_s * xi[0];
  float o[16];
  // the block's 64 x 64 elements lie in one 256 x 256 tile: one of the K-split last round (see bwd_dw_tail_kernel)?
  int tt = -1;
  if (tl.tile0 >= 0) {
    const int rt = blockIdx.y >> 2, ct = blockIdx.x >> 2, g8 = ct >> 3, gw = (CT - 8 * g8) < 8 ? (CT - 8 * g8) : 8;
    tt = g8 * 8 * RT + rt * gw + (ct - 8 * g8) - tl.tile0;       // (tile_from_index the other way round)
  }
  if (tt >= 0) {
    const int g0 = (tt * tl.kp) / tl.share, g1 = ((tt + 1) * tl.kp - 1) / tl.share;
    const float* src = tl.buf + (size_t)tt * 65536 + (j0 & 255) * 256 + (v & 255);
#pragma unroll
    for (int m = 0; m < 16; ++m) o[m] = 0.f;
    for (int g = g0; g <= g1; ++g) {                      // fixed order; the 16 loads of a piece are in flight together
#pragma unroll
      for (int m = 0; m < 16; ++m) o[m] += src[(size_t)g * 65536 + m * 256];
    }
#pragma unroll
    for (int m = 0; m < 16; ++m) o[m] *= scale;
  } else {
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      float sum = dwacc[(int64_t)(j0 + m) * Vp + v];
      for (int q = 1; q < nparts; ++q) sum += dwacc[q * part_stride + (int64_t)(j0 + m) * Vp + v];   // fixed order
      o[m] = sum * scale;
    }
  }
  const int s0 = segoff[v], L = segoff[v + 1] - s0;
  if (L >= LONG_SEG) {
    int nch, len;
    long_chunks(L, nch, len);
    for (int c = 0; c < nch; ++c) {                       // fixed order
      const float* ls = longsum + (int64_t)(longbase[v] + c) * dq + j0;
#pragma unroll
      for (int m = 0; m < 16; ++m) o[m] -= ls[m] * x_s;
    }
  } else if (L > 0) {
    for (int n = 0; n < L; ++n) {
      const int e = perm[s0 + n];                         // entry id k * Np + i
      const float h = hcoef[e] * x_s;
      const v4i raw = *reinterpret_cast<const v4i*>(xq + (int64_t)(e % Np) * ldx + j0);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const uint32_t w = (uint32_t)raw[m];
        o[4 * m + 0] -= h * e4m3_to_float<0>(w);
        o[4 * m + 1] -= h * e4m3_to_float<1>(w);
        o[4 * m + 2] -= h * e4m3_to_float<2>(w);
        o[4 * m + 3] -= h * e4m3_to_float<3>(w);
      }
    }
  }
#pragma unroll
  for (int m = 0; m < 16; ++m)
    if (j0 + m < d) Elem<T>::store(dw + (int64_t)(j0 + m) * dw_ld + v, o[m]);
}

}  // namespace sce
