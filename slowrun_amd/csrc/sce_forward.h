// Forward kernels: row-boost sample, the logit-tile walk with its epilogues, combination of the vocabulary splits,
// mean reduction (internal header).
// Part of the one translation unit sce_kernels.hip, which includes it after the headers it builds on.
#pragma once

namespace sce {

// ------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------
struct FwdParams {
  const uint8_t* xq;       // [Np][dp]
  const uint8_t* wqt;      // [Vp][dp]
  float4* partials;        // [S][Np]: sum exp(z - cap), max u, argmax u (bits), unused
  const int64_t* targets;  // (N,)
  float* s_uy;             // [n_predict][Np]: raw logit u at the target of (offset, row): from fwd_sample_kernel (PRE), else written by the workgroup that meets it
  uint8_t* ghat_t;         // EMIT: G, all Np rows, tile by tile (kbv blocks of 128 columns per tile of 256 rows)
  uint32_t* gexp;          // EMIT: its block exponents [Vp / 128][kbw]
  const float* lam;        // EMIT: exponent boost of every row
  int64_t ignore_index;
  int64_t dp, ldx;         // K extent and row stride of xq / wqt
  int64_t kbw, kbv;        // blocks of 128 rows (the exponents' row stride) and of 128 columns
  int N, V, Np, RT, CT, S, n_predict;      // V: columns that take part; CT: column tiles walked (EMIT: all of Vp / 256)
  float sc;                // x_s * w_s
  float k1;                // x_s * w_s * 2 log2(e) / cap : exp2(acc * k1) = e^{2u/cap}
  float ic2;               // 1 / c2, c2 = -2 cap log2(e): e^{z - cap} = exp2(c2 / (1 + e^{2u/cap}))
  float c2;
  float em2cap;            // e^{-2 cap}: what a logit of -inf adds to the sum of e^{z - cap}
  const DevConsts* dc;     // non-NULL: sc and k1 come from here (a scale lives on the device)
  int want_argmax;         // the caller asks for the rows' argmax: the column of the running maximum is tracked
};

// Per 256 x 256 tile and per row a lane owns: add up e^{z - cap} over its 64 columns and keep the
// largest raw accumulator.  z is bounded by +-cap, so no running maximum is needed for the sum:
//   t = tanh(u/cap) = 1 - 2/(E + 1), E = e^{2u/cap};   e^{z - cap} = exp2(c2 / (E + 1)).
// The column of the maximum is looked up only on the (rare, after the first tiles) occasion that
// a tile raises a row's running maximum.
template <bool EDGE>
__device__ __forceinline__ void fwd_epilogue(const v16f (&acc)[4][4], const FwdParams& p, int vbase,
                                             float (&sum)[4], float (&amax)[4], int (&uarg)[4]) {
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    float tmax = -INFINITY, s = 0.f;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int vo = a * 32 + 8 * (r >> 2) + (r & 3);
        float x = acc[a][b][r];
        // z - cap = c2 / (1 + e^{2u/cap}) in units of log2: the reciprocal of (1 + e) / c2 gives it in one step
        float pt = fast_exp2(fast_rcp(fmaf(fast_exp2(x * p.k1), p.ic2, p.ic2)));
        if (EDGE) {
          if (vo >= p.V - vbase) { pt = 0.f; x = -INFINITY; }
        }
        s += pt;
        tmax = fmaxf(tmax, x);
      }
    }
    sum[b] += s;
    if (p.want_argmax && __builtin_amdgcn_ballot_w64(tmax > amax[b]) != 0) {
      if (tmax > amax[b]) {
        int targ = 0x7fffffff;
#pragma unroll
        for (int a = 3; a >= 0; --a) {
#pragma unroll
          for (int r = 15; r >= 0; --r) {
            const int vo = a * 32 + 8 * (r >> 2) + (r & 3);
            if (acc[a][b][r] == tmax && (!EDGE || vo < p.V - vbase)) targ = vo;   // descending scan: lowest column wins
          }
        }
        amax[b] = tmax;
        uarg[b] = vbase + targ;
      }
    }
  }
}

__device__ __forceinline__ bool target_valid(const int64_t* __restrict__ targets, int64_t ignore_index, int i, int N, int V) {
  if (i >= N) return false;
  const int64_t y = targets[i];
  return (y != ignore_index) && y >= 0 && y < V;
}

// The raw logit at a row's targets, taken from the accumulators of the tile that holds the target column, so that z_y
// and lse come from the same numbers: the fp8 matrix instruction sums with less than fp32 care (it aligns its 64 products
// to the largest and drops what falls below about 2^-12 of it: about 2e-5 low on a sum of like-signed terms at K = 2560), and a z_y from a separate fp32 dot product would leave that bias in z_y - lse, i.e. in
// 1 - p_y, where rows the model is sure of cannot afford it.  tgt (LDS): [4 offsets][TGT_STRIDE rows] target column or
// -1, already at the wave's first row.  A lane looks at its four rows; the 64-way select runs only when some lane of
// the wave has a hit (a few per cent of the tiles) -- but the compiler moves the row block's 64 accumulators out of the
// accumulation registers around every offset's lookup, hit or not, which is why the fp8 kernels take their target
// logits from fwd_sample_kernel where they can (PRE) and this function serves the rest: the bf16 kernel, and W_q^T
// beyond that kernel's reach.
// STORE: the logit goes to s_uy_tile[offset][row] (global).
// KNOCK: the accumulator of the target is then set to -inf, for the dlogits epilogue that follows: the target takes
//        no part in the stored dlogits (its column is handled in fp32, see bwd_prep_kernel) and must not set the
//        exponent of its block either -- a row the model is sure of would push its own other columns, and its
//        neighbours', out of the 8 bits.
// B0, B1: the row blocks [B0, B1) only.
// STATS: with KNOCK, the row statistics (stat, as in form_dlogits) take the target's share here: e^{z_y - cap} into the
//        sum, and the running maximum / argmax.
template <bool STORE, bool KNOCK, bool STATS, int TGT_STRIDE, int B0 = 0, int B1 = 4>
__device__ __forceinline__ void take_target_logits(v16f (&acc)[4][4], const int* tgt, int n_predict, int col0, int rowbase,
                                                   float sc, float* s_uy_tile, int Np, float* stat, float k1, float ic2, float em2cap) {
  const int lane = lane_id(), half = lane >> 5;
#pragma unroll
  for (int b = B0; b < B1; ++b) {
    const int row = b * 32 + (lane & 31);
    float xk[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < n_predict; ++k) {
      const int y = tgt[k * TGT_STRIDE + row];
      const int rel = y - col0;                        // column within the wave's 128
      const bool hit = (unsigned)rel < 128u && ((rel >> 2) & 1) == half;
      if (__builtin_amdgcn_ballot_w64(hit) != 0) {
        if (hit) {
          const int idx = (rel >> 5) * 16 + ((rel >> 3) & 3) * 4 + (rel & 3);
          float x = 0.f;
          bool again = false;                          // an earlier offset of this row has the same target
          if (KNOCK) {
            for (int k2 = 0; k2 < k; ++k2)
              if (tgt[k2 * TGT_STRIDE + row] == y) { again = true; x = xk[k2]; }
          }
          if (!again) {
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                x = (idx == a * 16 + r) ? acc[a][b][r] : x;
                if (KNOCK) acc[a][b][r] = (idx == a * 16 + r) ? -INFINITY : acc[a][b][r];
              }
            if (KNOCK && STATS) {
              // (the -inf left behind reads as z = -cap to the epilogue that follows, which will add e^{-2 cap} for it)
              stat[(0 + b) * NTHREADS] += fast_exp2(fast_rcp(fmaf(fast_exp2(x * k1), ic2, ic2))) - em2cap;
              const float amax = stat[(4 + b) * NTHREADS];
              if (x > amax || (x == amax && y < __float_as_int(stat[(8 + b) * NTHREADS]))) {
                stat[(4 + b) * NTHREADS] = x;
                stat[(8 + b) * NTHREADS] = __int_as_float(y);
              }
            }
          }
          xk[k] = x;
          // (the lane index is taken anew: an address kept from outside the branch stays live across the main loop and is spilled)
          if (STORE) s_uy_tile[(int64_t)k * Np + rowbase + b * 32 + (lane_id() & 31)] = x * sc;
        }
      }
    }
  }
}

// The exponent boost of every row: lam_i = floor(-log2 Z^_i), Z^_i an estimate of the row's softmax sum Z_i = sum_v e^{z_iv - cap}
// made before the forward kernel starts, so that the stored value D 2^lam is close to the row's probabilities
// (times 1 - t^2) whatever the level of its logits.  Two tiles of logits go into it (one workgroup per row tile):
//   * 256 columns from the middle of the vocabulary, for the level of the row's bulk: V times m_i, the smallest of the
//     means of e^{z - cap} over 16 groups of 16 columns (the smallest, so that a few peaks inside the sample do not
//     pass for the level of the row);
//   * the 256 columns that are the targets of the tile's own rows (the rows of W^T gathered by the tile loader): the
//     row's own target -- where a confident row that is right has most of its sum -- and the tokens around it in the
//     text, where a language model's rows tend to have their other peaks.
// Every single e^{z - cap} is a lower bound of the sum, so Z^_i = max(V m_i, largest value seen in either tile).  What
// the estimate cannot see is a peak in a column that is in neither tile: such a row is boosted too far by the share
// of that peak in its sum (see form_dlogits for what that costs the rows that share its blocks).
// A row that has no valid target at all takes no part in the backward pass (its weight is zero): it gets the lowest
// boost, so that whatever its logits hold cannot set the exponent of a block.
//
// GATHER = false: the first tile only (the gathered rows' offsets would not fit the loader's 32 bits: W_q^T of 4 GiB or more).
// GATHER = true also leaves the target logits of the tile's rows in s_uy, for the forward kernel that follows: u[i, y_{i+k}]
// is element (i, i + k) of the gathered tile, computed by the same instructions in the same order as the forward
// kernel will compute it (bit for bit: that kernel recognises the entry by its value).  The offsets k >= 1 of the
// tile's last rows point at targets of the next tile's rows: those (at most three) ride as the last columns of the
// first tile, in place of the sampled columns there.
constexpr int SMEM_SAMPLE = SMEM_BYTES + 2 * 256 * 4 + 8 * 256 * 4;      // the K slots, the gathered rows, the rows without a target, the first tile's results
// BOOST = false (with GATHER): the target logits only, for a forward pass that emits nothing (the first tile is then
// computed only for the sake of its last columns, i.e. with more than one offset).
template <bool GATHER, bool BOOST = true>
__global__ __launch_bounds__(256) void fwd_sample_kernel(FwdParams p_in, int ct, float* __restrict__ lam_out) {
  static_assert(GATHER || BOOST, "nothing to do");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  FwdParams p = p_in;
  if (p.dc) { p.sc = p.dc->sc; p.k1 = p.dc->k1; }
  const int rt = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wa = wave >> 1, wb = wave & 1;
  int* rows = reinterpret_cast<int*>(smem + SMEM_BYTES);         // [256]: the row of W^T that column j of a tile is
  int* dead = rows + 256;                                        // [256]: row j has no valid target
  const int ntail = GATHER ? p.n_predict - 1 : 0;                // columns 256 - ntail .. 255 of the first tile: the next rows' targets
  auto column_of = [&](int64_t y) { return (y != p.ignore_index && y >= 0 && y < p.V) ? (int)y : 0; };
  if (GATHER) {
    // (a row without a target stands in with column 0: any column of the vocabulary gives a valid lower bound of the sum)
    const int t = threadIdx.x, j = t - (256 - ntail), row = rt * 256 + 256 + j;
    rows[t] = j < 0 ? ct * 256 + t : column_of(row < p.N ? p.targets[row] : p.ignore_index);
    __syncthreads();
  }
  // the targets of the thread's row are fetched before the first main loop, which hides the wait
  int64_t yraw[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int row = rt * 256 + (int)threadIdx.x;
    yraw[k] = (k < p.n_predict && row + k < p.N && row < p.N) ? p.targets[row + k] : p.ignore_index;
  }
  v16f acc[4][4];
  const bool first_tile = BOOST || ntail > 0;
  if (first_tile) {
    if (GATHER) mfma_mainloop(p.wqt, p.ldx, p.xq + (int64_t)rt * 256 * p.ldx, p.ldx, (int)(p.dp / BK), smem, acc, 0, 0, wave, NoHook(), 0, 0, nullptr, rows);
    else mfma_mainloop(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, p.xq + (int64_t)rt * 256 * p.ldx, p.ldx, (int)(p.dp / BK), smem, acc, 0, 0, wave);
  }
  {
    bool any = false;
#pragma unroll
    for (int k = 0; k < 4; ++k) any = any || (yraw[k] != p.ignore_index && yraw[k] >= 0 && yraw[k] < p.V);
    rows[threadIdx.x] = column_of(yraw[0]);
    dead[threadIdx.x] = !any;
  }
  const int lane = lane_id();
  if (GATHER && first_tile) {
    // columns 252 .. 255 are registers 12 .. 15 of A block 3 in the upper half-wave of the waves with wa = 1; rows 224 .. 255
    // are B block 3 of the waves with wb = 1
    const int i = 224 + (lane & 31);
    const bool mine = wave == 3 && lane >= 32;
#pragma unroll
    for (int r = 12; r < 16; ++r) {
      const int k = 256 + (252 + (r & 3) - (256 - ntail)) - i;       // the offset of row i that this column serves
      if (mine && 252 + (r & 3) >= 256 - ntail && k >= 1 && k < p.n_predict) p.s_uy[(int64_t)k * p.Np + rt * 256 + i] = acc[3][3][r] * p.sc;
    }
  }
  const int vlim = min(p.V - ct * 256, 256 - ntail), vloc0 = wa * 128 + 4 * (lane >> 5);
  float gmin[4], top[4];                                         // top: the largest logit seen (in the accumulator's units)
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    gmin[b] = INFINITY; top[b] = -INFINITY;
    if (!BOOST) continue;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      float sum = 0.f, cnt = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pt = fast_exp2(fast_rcp(fmaf(fast_exp2(acc[a][b][r] * p.k1), p.ic2, p.ic2)));
        const bool live = vloc0 + a * 32 + 8 * (r >> 2) + (r & 3) < vlim;
        sum += live ? pt : 0.f;
        cnt += live ? 1.f : 0.f;
        top[b] = live ? fmaxf(top[b], acc[a][b][r]) : top[b];
      }
      if (cnt > 0.f) gmin[b] = fminf(gmin[b], sum / cnt);
    }
  }
  if (GATHER && p.n_predict > 0) {      // (a condition the compiler cannot decide: merged into one block, the code of the two main loops is spilled)
    // the first tile's results wait in LDS: there is no register for them in the main loop
    float* keep = reinterpret_cast<float*>(smem + SMEM_BYTES + 2048) + threadIdx.x;
#pragma unroll
    for (int b = 0; b < 4; ++b) { keep[b * 256] = gmin[b]; keep[(4 + b) * 256] = top[b]; }
    __syncthreads();
    mfma_mainloop(p.wqt, p.ldx, p.xq + (int64_t)rt * 256 * p.ldx, p.ldx, (int)(p.dp / BK), smem, acc, 0, 0, wave, NoHook(), 0, 0, nullptr, rows);
    keep = reinterpret_cast<float*>(smem + SMEM_BYTES + 2048) + wave * 64 + lane_id();
#pragma unroll
    for (int b = 0; b < 4; ++b) { gmin[b] = keep[b * 256]; top[b] = keep[(4 + b) * 256]; }
    if (BOOST) {
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int r = 0; r < 16; ++r) top[b] = fmaxf(top[b], acc[a][b][r]);
    }
    // The band 0 <= column - row < n_predict lies in the 32 x 32 blocks on the diagonal and right of it: blocks (a, b) with
    // a - b = 0 or 1 of the waves with wa = wb, block (0, 3) of the wave with wa = 1, wb = 0.  (Stores under a lane
    // condition, no branches around the accumulators.)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int a = b; a < 5; ++a) {
        if (a > b + 1 && !(a == 4 && b == 3)) continue;
        const int aa = a & 3;                                    // (a = 4: A block 0 of the waves one to the right)
        const bool mine = a < 4 ? wa == wb : (wa == 1 && wb == 0);
        const int i = wb * 128 + b * 32 + (lane_id() & 31);      // (the lane index taken anew: what is prepared before the main loop is spilled across it)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int k = wa * 128 + aa * 32 + 8 * (r >> 2) + 4 * (lane_id() >> 5) + (r & 3) - i;
          if (mine && k >= 0 && k < p.n_predict) p.s_uy[(int64_t)k * p.Np + rt * 256 + i] = acc[aa][b][r] * p.sc;
        }
        __builtin_amdgcn_sched_barrier(0);      // (one block's accumulators at a time: all of them moved up front do not fit the registers)
      }
  }
  if (!BOOST) return;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    gmin[b] = fminf(gmin[b], __shfl_xor(gmin[b], 32));
    top[b] = fmaxf(top[b], __shfl_xor(top[b], 32));
  }
  float* red = reinterpret_cast<float*>(smem);          // free: the main loop has ended in every wave
  if (wa == 1 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 4; ++b) { red[wb * 128 + b * 32 + lane] = gmin[b]; red[256 + wb * 128 + b * 32 + lane] = top[b]; }
  }
  __syncthreads();
  if (wa == 0 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float m = fminf(gmin[b], red[wb * 128 + b * 32 + lane]), u = fmaxf(top[b], red[256 + wb * 128 + b * 32 + lane]);
      const float peak = fast_exp2(fast_rcp(fmaf(fast_exp2(u * p.k1), p.ic2, p.ic2)));       // (u = -inf: e^{-2 cap})
      float l = floorf(-log2f(fmaxf((float)p.V * m, peak)));
      l = l > -64.f ? (l < 120.f ? l : 120.f) : -64.f;
      lam_out[rt * 256 + wb * 128 + b * 32 + lane] = dead[wb * 128 + b * 32 + lane] ? -64.f : (l == l ? l : 0.f);
    }
  }
}

// The target entries of the dlogits that a forward pass has emitted are set to zero: they take no part in D (their
// share goes into the one-hot coefficient in fp32, see bwd_prep_kernel).  One thread per row.
__global__ __launch_bounds__(256) void fwd_knock_kernel(uint8_t* __restrict__ ghat, int64_t kbv, const int64_t* __restrict__ targets,
                                                       int64_t ignore_index, int N, int V, int n_predict) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  for (int k = 0; k < n_predict; ++k) {
    if (!target_valid(targets, ignore_index, i + k, N, V)) continue;
    const int64_t y = targets[i + k];
    ghat[((int64_t)(i >> 8) * kbv + (y >> 7)) * BLOCKED_KSTEP + (i & 255) * BK + (y & 127)] = 0;
  }
}

// LDS of the forward kernel: the two K slots; the row statistics of the workgroup's walk (12 values per lane, and the boosts of
// its rows: kept in registers they are spilled around the main loop, and the reload -- a vector memory load -- makes the
// epilogue wait for the tile loads that were just put in flight for the next tile); the targets of the workgroup's 256 rows.
constexpr int FWD_STAT_OFF = SMEM_MAX - 4096 - 16 * 4 * NTHREADS;      // 12 statistics and the boosts of the lane's 4 rows
constexpr int FWD_TGT_OFF = SMEM_MAX - 4096;
constexpr int FWD_UY_OFF = FWD_STAT_OFF - 4096;                        // PRE: the target logits of the rows, laid out like the targets
constexpr int SMEM_FWD = SMEM_MAX;
static_assert(SMEM_BYTES <= FWD_UY_OFF, "K slots and row data overlap");

// EMIT: the epilogue also leaves the block-scaled dlogits of the tile in G (see form_dlogits), for a backward pass
// that does not compute the logits again.
// BF16 (without EMIT): bf16 operands, logits rounded to bf16 as the eager head's GEMM returns them (forward only).
// PRE: the target logits are in s_uy already (fwd_sample_kernel<true, .>) and this kernel does not look for them in
// its accumulators.  With EMIT the target entries go through the epilogue like any other, except that they are kept out
// of the block exponents (form_dlogits, EXCL), and fwd_knock_kernel clears their bytes of G afterwards.
template <bool EMIT, bool BF16 = false, bool PRE = false>
__global__ __launch_bounds__(256) void fwd_kernel(FwdParams p_in) {
  static_assert(!PRE || !BF16, "PRE is for the fp8 kernels");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  FwdParams p = p_in;
  if (p.dc) { p.sc = p.dc->sc; p.k1 = p.dc->k1; }
  int rt, s;
  if (!map_tile(blockIdx.x, p.RT, p.S, rt, s)) return;
  const int ct0 = (int)((int64_t)p.CT * s / p.S), ct1 = (int)((int64_t)p.CT * (s + 1) / p.S);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wa = wave >> 1, wb = wave & 1;
  {
    float* stat = reinterpret_cast<float*>(smem + FWD_STAT_OFF) + wave * 64 + lane_id();   // [12][256]: sum, amax, uarg of the 4 row blocks
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      stat[(0 + b) * NTHREADS] = 0.f;
      stat[(4 + b) * NTHREADS] = -INFINITY;
      stat[(8 + b) * NTHREADS] = __int_as_float(0x7fffffff);
      if (EMIT) stat[(12 + b) * NTHREADS] = p.lam[rt * 256 + wb * 128 + b * 32 + (lane_id() & 31)];
    }
    int* tgt = reinterpret_cast<int*>(smem + FWD_TGT_OFF);
    for (int e = threadIdx.x; e < p.n_predict * 256; e += NTHREADS) {
      const int i = rt * 256 + (e & 255) + (e >> 8);
      tgt[e] = ((e & 255) + rt * 256 < p.N && target_valid(p.targets, p.ignore_index, i, p.N, p.V)) ? (int)p.targets[i] : -1;
      if (PRE && EMIT) reinterpret_cast<float*>(smem + FWD_UY_OFF)[e] = p.s_uy[(int64_t)(e >> 8) * p.Np + rt * 256 + (e & 255)];
    }
  }
  __syncthreads();
  v16f acc[4][4];
  const uint8_t* Bg = p.xq + (int64_t)rt * 256 * p.ldx;
  const int KT = (int)(p.dp / BK);
  // of the workgroups that start together on this XCD, those with the same split share the W tiles, those with the same rt the X rows
  const int rot_a = 2 * (rt & 3), rot_b = s & 7;
  // the first K blocks of the next tile travel while the epilogue of this one runs (it does not touch the K slots)
  if (ct0 < ct1) mfma_prefetch(p.wqt + (int64_t)ct0 * 256 * p.ldx, p.ldx, Bg, p.ldx, smem, rot_a, rot_b, wave);
  for (int ct = ct0; ct < ct1; ++ct) {
    if (EMIT) mfma_mainloop<true, NoHook, BK, false, 0, false, true>(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, Bg, p.ldx, KT, smem, acc, rot_a, rot_b, wave);
    else mfma_mainloop<true, NoHook, BK, false, 0, BF16>(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, Bg, p.ldx, KT, smem, acc, rot_a, rot_b, wave);
    auto prefetch = [&]() {
      if (ct + 1 < ct1) mfma_prefetch(p.wqt + (int64_t)(ct + 1) * 256 * p.ldx, p.ldx, Bg, p.ldx, smem, rot_a, rot_b, wave);
    };
    if (!EMIT) prefetch();
    float* stat = reinterpret_cast<float*>(smem + FWD_STAT_OFF) + wave * 64 + lane_id();
    const int vbase = ct * 256 + wa * 128 + 4 * (lane_id() >> 5);
    const int* tgt = reinterpret_cast<const int*>(smem + FWD_TGT_OFF) + wb * 128;
    if (EMIT) {
      // The main loop has left 48 of the 64 MFMAs of its last pair of K blocks undone, those of row blocks 1 - 3; the pair
      // is still in LDS.  They are issued one at a time between the stages of the epilogues of row blocks 0 and 1, where
      // the matrix pipe would stand idle: during block 0's the 32 of blocks 1 and 2 (one at each of its 32 stage
      // boundaries), during block 1's the 16 of block 3.  Only then are the slots free for the next tile's first K blocks.
      DeferredTail deferred(smem, wa, wb);
      auto tail = [&](int b, int k) { deferred(acc, b, k); };
      const int vlim = p.V - ct * 256;
      // the wave's quadrant of G: tile of rows rt, block of columns 2 ct + wa, rows 128 wb on
      uint8_t* gq = p.ghat_t + ((int64_t)rt * p.kbv + 2 * ct + wa) * BLOCKED_KSTEP + wb * 128 * BK;
      const float* lam = reinterpret_cast<const float*>(smem + FWD_STAT_OFF) + 12 * NTHREADS + wave * 64;
      const int col0 = ct * 256 + wa * 128, row0 = rt * 256 + wb * 128;
      // (one code path for the epilogue: with a second one for the last tile of the vocabulary, each with its MFMAs, the
      // accumulators are spilled; columns that do not exist are struck out of the finished accumulators instead)
      const bool ragged = vlim < 256;
      uint32_t ew;
      if (PRE) {
        // which of the lane's values of row block b is a target of its row (one is looked for: two targets of a row in one
        // lane's 64 columns are the same column, or rare enough that the second may set an exponent): its known value
        const float* tuy = reinterpret_cast<const float*>(smem + FWD_UY_OFF) + wb * 128;
        auto target_value = [&](int b) {
          float v = __builtin_nanf("");
          for (int k = 0; k < p.n_predict; ++k) {
            const int rel = tgt[k * 256 + b * 32 + (lane_id() & 31)] - col0;
            if ((unsigned)rel < 128u && ((rel >> 2) & 1) == (lane_id() >> 5)) v = tuy[k * 256 + b * 32 + (lane_id() & 31)];
          }
          return v;
        };
        float xc[4];                                   // (looked up a row block ahead of their use: the LDS reads have time)
        if (ragged) strike_columns_beyond<0, 1>(acc, vlim, wa, stat, p.em2cap);
        xc[0] = target_value(0); xc[1] = target_value(1);
        ew = form_dlogits<true, NTHREADS, 64, 0, 1, decltype(tail)&, true>(acc, p.k1, p.c2, vbase, gq, wa, wb, stat, lam, p.want_argmax != 0, tail, xc, p.sc);
        if (ragged) strike_columns_beyond<1, 2>(acc, vlim, wa, stat, p.em2cap);
        xc[2] = target_value(2); xc[3] = target_value(3);
        ew |= form_dlogits<true, NTHREADS, 64, 1, 2, decltype(tail)&, true>(acc, p.k1, p.c2, vbase, gq, wa, wb, stat, lam, p.want_argmax != 0, tail, xc, p.sc);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // every wave has read its last fragment
        prefetch();
        if (ragged) strike_columns_beyond<2, 4>(acc, vlim, wa, stat, p.em2cap);
        NoHook none;
        ew |= form_dlogits<true, NTHREADS, 64, 2, 4, NoHook&, true>(acc, p.k1, p.c2, vbase, gq, wa, wb, stat, lam, p.want_argmax != 0, none, xc, p.sc);
      } else {
        if (ragged) strike_columns_beyond<0, 1>(acc, vlim, wa, stat, p.em2cap);
        take_target_logits<true, true, true, 256, 0, 1>(acc, tgt, p.n_predict, col0, row0, p.sc, p.s_uy, p.Np, stat, p.k1, p.ic2, p.em2cap);
        ew = form_dlogits<true, NTHREADS, 64, 0, 1>(acc, p.k1, p.c2, vbase, gq, wa, wb, stat, lam, p.want_argmax != 0, tail);
        if (ragged) strike_columns_beyond<1, 2>(acc, vlim, wa, stat, p.em2cap);
        take_target_logits<true, true, true, 256, 1, 2>(acc, tgt, p.n_predict, col0, row0, p.sc, p.s_uy, p.Np, stat, p.k1, p.ic2, p.em2cap);
        ew |= form_dlogits<true, NTHREADS, 64, 1, 2>(acc, p.k1, p.c2, vbase, gq, wa, wb, stat, lam, p.want_argmax != 0, tail);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // every wave has read its last fragment
        prefetch();
        if (ragged) strike_columns_beyond<2, 4>(acc, vlim, wa, stat, p.em2cap);
        take_target_logits<true, true, true, 256, 2, 4>(acc, tgt, p.n_predict, col0, row0, p.sc, p.s_uy, p.Np, stat, p.k1, p.ic2, p.em2cap);
        ew |= form_dlogits<true, NTHREADS, 64, 2, 4>(acc, p.k1, p.c2, vbase, gq, wa, wb, stat, lam, p.want_argmax != 0);
      }
      if (lane_id() == 0) p.gexp[(int64_t)(2 * ct + wa) * p.kbw + 2 * rt + wb] = ew;
    } else {
      float sum[4], amax[4];
      int uarg[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        sum[b] = stat[(0 + b) * NTHREADS]; amax[b] = stat[(4 + b) * NTHREADS]; uarg[b] = __float_as_int(stat[(8 + b) * NTHREADS]);
      }
      if (BF16) {
        // the GEMM of the eager head returns bf16: the logits are rounded once, in place, and everything after sees the rounded values
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = round_to_bf16_hw(acc[a][b][r]);
      }
      if (ct * 256 + 256 > p.V) fwd_epilogue<true>(acc, p, vbase, sum, amax, uarg);
      else fwd_epilogue<false>(acc, p, vbase, sum, amax, uarg);
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        stat[(0 + b) * NTHREADS] = sum[b]; stat[(4 + b) * NTHREADS] = amax[b]; stat[(8 + b) * NTHREADS] = __int_as_float(uarg[b]);
      }
    }
    if (!EMIT && !PRE) take_target_logits<true, false, false, 256>(acc, tgt, p.n_predict, ct * 256 + wa * 128, rt * 256 + wb * 128, p.sc, p.s_uy, p.Np, nullptr, 0.f, 0.f, 0.f);
  }
  float sum[4], amax[4];
  int uarg[4];
  const int lane = lane_id();
  float* stat = reinterpret_cast<float*>(smem + FWD_STAT_OFF) + wave * 64 + lane;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    sum[b] = stat[(0 + b) * NTHREADS]; amax[b] = stat[(4 + b) * NTHREADS]; uarg[b] = __float_as_int(stat[(8 + b) * NTHREADS]);
  }
  // the two half-waves hold different columns of the same rows
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const float s2 = __shfl_xor(sum[b], 32), um2 = __shfl_xor(amax[b], 32);
    const int ua2 = __shfl_xor(uarg[b], 32);
    sum[b] += s2;
    if (um2 > amax[b] || (um2 == amax[b] && ua2 < uarg[b])) { amax[b] = um2; uarg[b] = ua2; }
  }
  // waves wa = 0 and wa = 1 hold different columns of the same rows
  float4* red = reinterpret_cast<float4*>(smem);
  if (wa == 1 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 4; ++b) red[wb * 128 + b * 32 + lane] = make_float4(sum[b], amax[b], __int_as_float(uarg[b]), 0.f);
  }
  __syncthreads();
  if (wa == 0 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float4 o = red[wb * 128 + b * 32 + lane];
      const int ua2 = __float_as_int(o.z);
      sum[b] += o.x;
      if (o.y > amax[b] || (o.y == amax[b] && ua2 < uarg[b])) { amax[b] = o.y; uarg[b] = ua2; }
      p.partials[(int64_t)s * p.Np + rt * 256 + wb * 128 + b * 32 + lane] =
          make_float4(sum[b], amax[b] * p.sc, __int_as_float(uarg[b]), 0.f);
    }
  }
}

// What a block of 256 rows contributes to the mean loss: left by fwd_combine_kernel in the first 16 bytes of the
// block's own rows of the partial records (which it has consumed by then), summed by fwd_reduce_kernel.
struct BlockLoss {
  double sum;      // sum of lse_i - z[i, y_i] over the valid rows
  int32_t cnt;     // valid rows
  int32_t bad;     // targets outside [0, V) other than ignore_index
};
static_assert(sizeof(BlockLoss) == 16, "one float4 slot");

// one thread per row: fold the V-splits, write lse / loss / argmax and the saved row statistics
__global__ __launch_bounds__(256) void fwd_combine_kernel(float4* __restrict__ partials, int S, int N, int Np, int V,
                                                         const int64_t* __restrict__ targets, int64_t ignore_index, float cap,
                                                         const float* __restrict__ mtp_weights, int n_predict,
                                                         float* __restrict__ s_lse, float* __restrict__ s_umax,
                                                         float* __restrict__ s_zy, float* __restrict__ losses,
                                                         float* __restrict__ lse_out, int32_t* __restrict__ argmax_out) {
  __shared__ double ssum[256];
  __shared__ int scnt[256], sbad[256];
  const int t = threadIdx.x, i = blockIdx.x * 256 + t;      // the grid covers Np = 256 * gridDim.x rows exactly
  double term = 0.0;
  int cnt = 0, bad = 0;
  if (i >= N) {
    s_lse[i] = 0.f; s_umax[i] = 0.f;
    for (int k = 0; k < n_predict; ++k) s_zy[(int64_t)k * Np + i] = 0.f;
  } else {
    float sum = 0.f, umax = -INFINITY;
    int uarg = 0x7fffffff;
    for (int s = 0; s < S; ++s) {
      const float4 o = partials[(int64_t)s * Np + i];
      const int ua = __float_as_int(o.z);
      sum += o.x;
      if (o.y > umax || (o.y == umax && ua < uarg)) { umax = o.y; uarg = ua; }
    }
    const float lse = cap + logf(sum);
    s_lse[i] = lse; s_umax[i] = umax;
    // the forward kernel left the raw logit at each target that takes part: z_y = cap tanh(u_y / cap) replaces it (0 for the others);
    // loss_i = sum_k w_k (lse_i - z[i, y_{i+k}]) over the offsets that take part (tiny/cuda_kernels.py:226-240)
    float l = 0.f;
    for (int k = 0; k < n_predict; ++k) {
      float zy = 0.f;
      if (target_valid(targets, ignore_index, i + k, N, V)) {
        zy = cap * tanhf(s_zy[(int64_t)k * Np + i] / cap);
        l += (mtp_weights ? mtp_weights[k] : 1.0f) * (lse - zy);
      }
      s_zy[(int64_t)k * Np + i] = zy;
    }
    if (losses) losses[i] = l;
    if (lse_out) lse_out[i] = lse;
    if (argmax_out) argmax_out[i] = (uarg == 0x7fffffff) ? 0 : uarg;
    const int64_t y = targets[i];
    if (y != ignore_index) {
      if (y < 0 || y >= V) bad = 1;
      else { term = (double)(lse - s_zy[i]); cnt = 1; }
    }
  }
  ssum[t] = term; scnt[t] = cnt; sbad[t] = bad;
  __syncthreads();               // also: every row of this block has read its partial records
  for (int w = 128; w > 0; w >>= 1) {
    if (t < w) { ssum[t] += ssum[t + w]; scnt[t] += scnt[t + w]; sbad[t] += sbad[t + w]; }
    __syncthreads();
  }
  if (t == 0) {
    BlockLoss bl;
    bl.sum = ssum[0]; bl.cnt = scnt[0]; bl.bad = sbad[0];
    *reinterpret_cast<BlockLoss*>(partials + (int64_t)blockIdx.x * 256) = bl;
  }
}

// What a forward call was asked for, as far as the matching backward call must have been asked the same: left in the header
// of the saved state (HDR_MODE_OFF bytes in) by fwd_reduce_kernel and compared by bwd_prep_kernel.  A backward call whose
// flags differ would read dlogits that were never written, or mask other columns: it gets NaN gradients instead.
struct CallMode {
  int32_t emit, vocab_limit, n_predict, cap_bits;
};
constexpr int HDR_MODE_OFF = 64;
static inline CallMode call_mode(bool emit, int vocab_limit, int n_predict, float cap) {
  CallMode m;
  m.emit = emit ? 1 : 0; m.vocab_limit = vocab_limit; m.n_predict = n_predict;
  memcpy(&m.cap_bits, &cap, 4);
  return m;
}

// single workgroup: n_valid, number of out-of-range targets, mean loss from the per-block sums (fixed order)
__global__ __launch_bounds__(1024) void fwd_reduce_kernel(const float4* __restrict__ partials, int nblk,
                                                         int32_t* __restrict__ hdr, float* __restrict__ loss_out,
                                                         int32_t* __restrict__ nvalid_out, CallMode mode) {
  __shared__ double ssum[1024];
  __shared__ int scnt[1024], sbad[1024];
  const int t = threadIdx.x;
  double acc = 0.0;
  int cnt = 0, bad = 0;
  for (int b = t; b < nblk; b += 1024) {
    const BlockLoss bl = *reinterpret_cast<const BlockLoss*>(partials + (int64_t)b * 256);
    acc += bl.sum; cnt += bl.cnt; bad += bl.bad;
  }
  ssum[t] = acc; scnt[t] = cnt; sbad[t] = bad;
  __syncthreads();
  for (int w = 512; w > 0; w >>= 1) {
    if (t < w) { ssum[t] += ssum[t + w]; scnt[t] += scnt[t + w]; sbad[t] += sbad[t + w]; }
    __syncthreads();
  }
  if (t == 0) {
    hdr[0] = scnt[0]; hdr[1] = sbad[0];
    const float mean = (float)(ssum[0] / (double)scnt[0]);   // 0/0 = NaN, as F.cross_entropy gives
    reinterpret_cast<float*>(hdr)[2] = mean;
    if (loss_out) *loss_out = mean;
    if (nvalid_out) { nvalid_out[0] = scnt[0]; nvalid_out[1] = sbad[0]; }
    *reinterpret_cast<CallMode*>(reinterpret_cast<uint8_t*>(hdr) + HDR_MODE_OFF) = mode;
  }
}

}  // namespace sce
