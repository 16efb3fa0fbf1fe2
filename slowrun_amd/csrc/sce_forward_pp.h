// The opt-in ping-pong forward kernel: epilogue units and kernel on top of pingpong_walk (internal header).
// Part of the one translation unit sce_kernels.hip, which includes it after the headers it builds on.
#pragma once

namespace sce {

// ------------------------------------------------------------------------------------------
// forward, ping-pong walk (sce_pingpong.h): the dlogits epilogue of one half-tile runs beside the MFMAs of the next
// ------------------------------------------------------------------------------------------
// LDS: the ring; a 2 KB staging block per wave index (the two groups never stage at the same time: their epilogues
// are a barrier apart); the boosts of the 256 rows; their targets.
constexpr int PP_STAGE_OFF = PP_RING;                       // [4][32 v][64 i] bytes
constexpr int PP_LAM_OFF = PP_STAGE_OFF + 4 * 2048;         // [256] floats
constexpr int PP_TGT_OFF = PP_LAM_OFF + 1024;               // [4 offsets][256] ints
constexpr int SMEM_FWD_PP = PP_TGT_OFF + 4096;
static_assert(SMEM_FWD_PP <= SMEM_MAX, "LDS of the ping-pong forward kernel");

// The epilogue of a 128 (v) x 64 (i) wave tile in 19 units: the rows' targets, the exponent of each of the two 32-row
// blocks, then the 128 values of a lane eight at a time; after every 32 columns (4 units) the 32 x 64 bytes staged in LDS
// leave for G^T as 64-byte runs.  The arithmetic is that of form_dlogits.  The row statistics stay in registers: sum of
// e^{z - cap}, largest raw logit and its column, for the lane's two rows.
// The accumulators are only read.  (Setting the targets' accumulators to -inf, as the one-wave-per-SIMD kernel does,
// makes the compiler rebuild the 16-register tuples in new registers, and the tile no longer fits.)  Instead a lane
// remembers which of its values are targets (kidx) and how large the largest of them is (tx); a target counts in the row
// statistics like any other column, stays out of the block's exponent (a second pass over the block, needed only when
// a target is the block's largest value in some lane) and is stored as zero.  Columns beyond V (last tile of a row)
// are left out of everything by the same slower paths.
// ARGMAX: the rows' largest raw logit and its column are kept as well (only a caller that asks for the argmax needs
// them; finding the column costs about as much as a sixth of the rest of the epilogue).
template <bool ARGMAX>
struct FwdPPEpi {
  static constexpr int UNITS = 19;
  struct P {            // the few fields of FwdParams the units use, by value: all of them stay in scalar registers
    float* s_uy; uint8_t* ghat_t; uint32_t* gexp;
    int64_t kbw;
    int V, Np, n_predict;
    float sc, k1, ic2, c2;
  } p;
  uint8_t* smem;
  int rt, h0, wi;
  float sum[2], amax[2];
  int uarg[2];
  float cs[2], ssum[2];
  uint32_t ew;
  int kidx[2][4];        // register index (a * 16 + r) of the target of (row block, offset) in this tile, or -1
  float tx[2];           // largest raw logit among the lane's targets in the row block
  bool any[2];           // some lane of the wave has a target in the row block (uniform)
  int ty[2];             // target (first offset) of the lane's row in each row block, or -1: the same for every tile of the walk
  float lamv[2];         // exponent boost of those rows
  uint32_t sel1, sel2;   // byte selectors of the lane's part in the 4 x 4 transposes
  uint32_t stage_at;     // LDS address of the lane's dword in row 0 of the wave's staging block
  __device__ __forceinline__ FwdPPEpi(const FwdParams& q, uint8_t* smem_, int rt_, int h0_, int wi_) : smem(smem_), rt(rt_), h0(h0_), wi(wi_) {
    {
      const int lane = lane_id(), k = lane & 3;
      sel1 = (k & 1) ? 0x03070105u : 0x06020400u;
      sel2 = (k & 2) ? 0x03020706u : 0x05040100u;
      stage_at = (uint32_t)(PP_STAGE_OFF + wi * 2048 + (4 * (lane >> 5) + k) * 64 + (lane & 28));
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        ty[b] = reinterpret_cast<const int*>(smem + PP_TGT_OFF)[wi * 64 + b * 32 + (lane & 31)];
        lamv[b] = reinterpret_cast<const float*>(smem + PP_LAM_OFF)[wi * 64 + b * 32 + (lane & 31)];
      }
    }
    p.s_uy = q.s_uy; p.ghat_t = q.ghat_t; p.gexp = q.gexp; p.kbw = q.kbw; p.V = q.V; p.Np = q.Np; p.n_predict = q.n_predict;
    p.sc = q.sc; p.k1 = q.k1; p.ic2 = q.ic2; p.c2 = q.c2;
    sum[0] = sum[1] = 0.f; amax[0] = amax[1] = -INFINITY; uarg[0] = uarg[1] = 0x7fffffff;
    begin();
  }
  // start of an epilogue: what the units hand to each other carries nothing over from the previous tile (so these
  // registers are free while the wave accumulates)
  __device__ __forceinline__ void begin() {
    cs[0] = cs[1] = ssum[0] = ssum[1] = 0.f; ew = 0;
    tx[0] = tx[1] = -INFINITY; any[0] = any[1] = false;
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int k = 0; k < 4; ++k) kidx[b][k] = -1;
  }
  template <int B>
  __device__ __forceinline__ bool is_target(int c) const {      // (no short-circuit: four compares, not four branches)
    return (int)(kidx[B][0] == c) | (int)(kidx[B][1] == c) | (int)(kidx[B][2] == c) | (int)(kidx[B][3] == c);
  }
  // column (within the tile) of value (a, r)
  __device__ __forceinline__ int column(int a, int r) const { return a * 32 + 8 * (r >> 2) + 4 * (lane_id() >> 5) + (r & 3); }

  // The raw logits at the rows' targets, as take_target_logits takes them.
  __device__ __forceinline__ void targets(const v16f (&acc)[4][2], int h) {
    const int half = lane_id() >> 5;
    const int col0 = h * 128;
    const int* tgt = reinterpret_cast<const int*>(smem + PP_TGT_OFF);
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int row = wi * 64 + b * 32 + (lane_id() & 31);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (k < p.n_predict) {
          const int y = k == 0 ? ty[b] : tgt[k * 256 + row];
          const int rel = y - col0;
          const bool hit = (unsigned)rel < 128u && ((rel >> 2) & 1) == half;
          if (__builtin_amdgcn_ballot_w64(hit) != 0) {
            any[b] = true;
            if (hit) {
              const int idx = (rel >> 5) * 16 + ((rel >> 3) & 3) * 4 + (rel & 3);
              float x = 0.f;
#pragma unroll
              for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) x = (idx == a * 16 + r) ? acc[a][b][r] : x;
              kidx[b][k] = idx;
              tx[b] = fmaxf(tx[b], x);
              float* dst = p.s_uy + (int64_t)k * p.Np + rt * 256 + wi * 64 + b * 32 + (lane_id() & 31);
              const float xs = x * p.sc;
              asm volatile("global_store_dword %0, %1, off" ::"v"(dst), "v"(xs) : "memory");
            }
          }
        }
      }
    }
  }

  // EDGE: the tile reaches beyond V (the last tile of a row only)
  template <int B, bool EDGE>
  __device__ __forceinline__ void block_exponent_v(const v16f (&acc)[4][2], int h) {
    float k1 = p.k1;
    asm volatile("" : "+v"(k1));       // (see values8)
    int vlim = p.V - h * 128;
    if (EDGE) asm volatile("" : "+v"(vlim));      // (keeps the 64 comparisons with it where they are: hoisted, their lane masks overflow the scalar registers)
    // the largest of the lane's 64 values: for the row's running maximum, and for the exponent
    float tmax = -INFINITY;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, (EDGE && column(a, r) >= vlim) ? -INFINITY : acc[a][B][r]);
    // running maximum and its column (a target is a column like any other here)
    if (ARGMAX && __builtin_amdgcn_ballot_w64(tmax >= amax[B] && tmax > -INFINITY) != 0) {
      if (tmax >= amax[B] && tmax > -INFINITY) {
        int targ = 0x7fffffff;
#pragma unroll
        for (int a = 3; a >= 0; --a)
#pragma unroll
          for (int r = 15; r >= 0; --r) {        // descending scan: lowest column wins
            bool ok = acc[a][B][r] == tmax;
            if (EDGE) ok = (int)ok & (int)(column(a, r) < vlim);
            targ = ok ? a * 32 + 8 * (r >> 2) + (r & 3) : targ;
          }
        const int col = h * 128 + 4 * (lane_id() >> 5) + targ;
        if (targ != 0x7fffffff && (tmax > amax[B] || col < uarg[B])) { amax[B] = tmax; uarg[B] = col; }
      }
    }
    // the exponent comes from the largest value that is stored: in a lane whose largest value is a target, once more without
    if (any[B]) {
      if (__builtin_amdgcn_ballot_w64(tx[B] >= tmax) != 0) {
        tmax = -INFINITY;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            bool out = is_target<B>(a * 16 + r);
            if (EDGE) out = (int)out | (int)(column(a, r) >= vlim);
            tmax = fmaxf(tmax, out ? -INFINITY : acc[a][B][r]);
          }
      }
    }
    const float lamb = lamv[B];
    const float lg = wave_max_dpp(fmaf(p.c2, fast_rcp(1.0f + fast_exp2(tmax * k1)), lamb));
    const float sb = floorf(8.8f - lg);
    cs[B] = sb + 2.0f + lamb;
    ssum[B] = 0.f;
    if (B == 0) ew = (uint32_t)(127 - (int)sb); else ew |= (uint32_t)(127 - (int)sb) << 8;
  }
  template <int B>
  __device__ __forceinline__ void block_exponent(const v16f (&acc)[4][2], int h) {
    if (p.V - h * 128 < 128) block_exponent_v<B, true>(acc, h);
    else block_exponent_v<B, false>(acc, h);
  }

  // eight of the lane's values of block (A, B): registers [G0, G0 + 8)
  template <int A, int B, int G0>
  __device__ __forceinline__ void values8(const v16f (&acc)[4][2], int h) {
    // The units depend on nothing that changes between the steps of the walk; without this the optimiser computes
    // all of them ahead of the loop of steps and keeps the results in scratch memory.
    float k1 = p.k1;
    asm volatile("" : "+v"(k1));
    const int vlim = p.V - h * 128;
    float rr[8], gg[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) rr[m] = fast_exp2(acc[A][B][G0 + m] * k1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 8; ++m) rr[m] = fast_rcp(rr[m] + 1.0f);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 8; ++m) gg[m] = fast_exp2(fmaf(p.c2, rr[m], cs[B]));
    __builtin_amdgcn_sched_barrier(0);
    if (vlim < 128) {       // columns beyond V count for nothing
      int vl = vlim;
      asm volatile("" : "+v"(vl));
#pragma unroll
      for (int m = 0; m < 8; ++m) gg[m] = column(A, G0 + m) >= vl ? 0.f : gg[m];
    }
#pragma unroll
    for (int m = 0; m < 8; ++m) ssum[B] += gg[m];
    if (any[B]) {           // a target is stored as zero (its share of the gradient is added in fp32 later)
      constexpr int C0 = A * 16 + G0;
      const bool mine = (int)((unsigned)(kidx[B][0] - C0) < 8u) | (int)((unsigned)(kidx[B][1] - C0) < 8u) | (int)((unsigned)(kidx[B][2] - C0) < 8u) |
                        (int)((unsigned)(kidx[B][3] - C0) < 8u);
      if (__builtin_amdgcn_ballot_w64(mine) != 0) {
#pragma unroll
        for (int m = 0; m < 8; ++m) gg[m] = is_target<B>(C0 + m) ? 0.f : gg[m];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 8; ++m) gg[m] *= rr[m] - rr[m] * rr[m];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const uint32_t w = cvt4_e4m3(gg[4 * q], gg[4 * q + 1], gg[4 * q + 2], gg[4 * q + 3]);
      // 4 x 4 byte transpose inside the quad: lane k ends up with column vloc + k, rows (i & ~3) .. +3
      const uint32_t p1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0xB1, 0xF, 0xF, true);     // lane ^ 1
      const uint32_t x = __builtin_amdgcn_perm(p1, w, sel1);
      const uint32_t p2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, true);     // lane ^ 2
      const uint32_t yv = __builtin_amdgcn_perm(p2, x, sel2);
      // lane k of a quad ends up with column 8 (G0 / 4 + q) + 4 (lane / 32) + k of block A, rows (i & ~3) .. +3 of block B
      *reinterpret_cast<uint32_t*>(smem + stage_at + 8 * (G0 / 4 + q) * 64 + B * 32) = yv;
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // the 32 columns of block A are staged: 32 rows of G^T, 64 bytes each (a wave reads only what it wrote itself)
  template <int A>
  __device__ __forceinline__ void store32(int h) {
    const int lane = lane_id();
    const uint8_t* TT = smem + PP_STAGE_OFF + wi * 2048;
    uint8_t* g = p.ghat_t + ((int64_t)(h >> 1) * p.kbw + 2 * rt + (wi >> 1)) * BLOCKED_KSTEP + ((h & 1) * 128 + A * 32) * BK + (wi & 1) * 64;
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int cidx = lane + 64 * n, row = cidx >> 2, col = (cidx & 3) * 16;
      // (Stores the compiler does not see: one that it knows of makes it wait, at the next unit, for every vector
      // memory operation in flight -- the tile loads included -- before it reuses the registers that held the data.)
      const v4i val = *reinterpret_cast<const v4i*>(TT + row * 64 + col);
      // (the no-ops: a store of more than 8 bytes reads its data registers for two more cycles, and the compiler, which
      // would otherwise keep the next instruction from overwriting them, does not know that this is one)
      asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" ::"v"(g + row * BK + col), "v"(val) : "memory");
    }
  }

  __device__ __forceinline__ void finish(int h) {
    sum[0] += ssum[0] * fast_exp2(-cs[0]);
    sum[1] += ssum[1] * fast_exp2(-cs[1]);
    if (lane_id() == 0) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(p.gexp) + ((int64_t)h * p.kbw + 2 * rt + (wi >> 1)) * 2 + (wi & 1);
      asm volatile("global_store_short %0, %1, off" ::"v"(dst), "v"(ew) : "memory");
    }
  }

  template <int Q>       // Q = 0..15: block A = Q / 4, B = (Q / 2) % 2, half = Q % 2
  __device__ __forceinline__ void values_unit(const v16f (&acc)[4][2], int h) {
    values8<Q / 4, (Q / 2) & 1, (Q & 1) * 8>(acc, h);
    if ((Q & 3) == 3) store32<Q / 4>(h);
    if (Q == 15) finish(h);
  }

  __device__ __forceinline__ void unit(int u, const v16f (&acc)[4][2], int j) {
    const int h = h0 + j;
    switch (u) {
      case 0: targets(acc, h); break;
      case 1: block_exponent<0>(acc, h); break;
      case 2: block_exponent<1>(acc, h); break;
#define SCE_PP_CASE(Q) case 3 + Q: values_unit<Q>(acc, h); break;
      SCE_PP_CASE(0) SCE_PP_CASE(1) SCE_PP_CASE(2) SCE_PP_CASE(3) SCE_PP_CASE(4) SCE_PP_CASE(5) SCE_PP_CASE(6) SCE_PP_CASE(7)
      SCE_PP_CASE(8) SCE_PP_CASE(9) SCE_PP_CASE(10) SCE_PP_CASE(11) SCE_PP_CASE(12) SCE_PP_CASE(13) SCE_PP_CASE(14) SCE_PP_CASE(15)
#undef SCE_PP_CASE
      default: break;
    }
  }
};

// One workgroup walks the half-tiles [CT2 s / S, CT2 (s + 1) / S) of row tile rt (CT2 = 2 CT) and leaves the same partial
// records and the same G^T, exponents and target logits as fwd_kernel<true>.
template <int LK, bool ARGMAX>
__global__ __launch_bounds__(PP_THREADS) void fwd_pp_kernel(FwdParams p_in) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  FwdParams p = p_in;
  if (p.dc) { p.sc = p.dc->sc; p.k1 = p.dc->k1; }
  int rt, s;
  if (!map_tile(blockIdx.x, p.RT, p.S, rt, s)) return;
  const int CT2 = 2 * p.CT;
  const int h0 = (int)((int64_t)CT2 * s / p.S), h1 = (int)((int64_t)CT2 * (s + 1) / p.S);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wi = wave & 3;
  {
    float* lam = reinterpret_cast<float*>(smem + PP_LAM_OFF);
    int* tgt = reinterpret_cast<int*>(smem + PP_TGT_OFF);
    for (int e = threadIdx.x; e < 256; e += PP_THREADS) lam[e] = p.lam[rt * 256 + e];
    for (int e = threadIdx.x; e < p.n_predict * 256; e += PP_THREADS) {
      const int i = rt * 256 + (e & 255) + (e >> 8);
      tgt[e] = ((e & 255) + rt * 256 < p.N && target_valid(p.targets, p.ignore_index, i, p.N, p.V)) ? (int)p.targets[i] : -1;
    }
  }
  __syncthreads();
  FwdPPEpi<ARGMAX> epi(p, smem, rt, h0, wi);
  pingpong_walk<FwdPPEpi<ARGMAX>, LK>(p.xq + (int64_t)rt * 256 * p.ldx, p.wqt + (int64_t)h0 * 128 * p.ldx, p.ldx, (int)(p.dp / BK), h1 - h0, smem, wave, epi);
  // the two half-waves hold different columns of the same rows; so do the two groups
  float sum[2], amax[2];
  int uarg[2];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const float s2 = __shfl_xor(epi.sum[b], 32), um2 = __shfl_xor(epi.amax[b], 32);
    const int ua2 = __shfl_xor(epi.uarg[b], 32);
    sum[b] = epi.sum[b] + s2; amax[b] = epi.amax[b]; uarg[b] = epi.uarg[b];
    if (um2 > amax[b] || (um2 == amax[b] && ua2 < uarg[b])) { amax[b] = um2; uarg[b] = ua2; }
  }
  __syncthreads();               // every wave is through with the ring
  const int lane = lane_id();
  float4* red = reinterpret_cast<float4*>(smem);
  if (wave >= 4 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 2; ++b) red[wi * 64 + b * 32 + lane] = make_float4(sum[b], amax[b], __int_as_float(uarg[b]), 0.f);
  }
  __syncthreads();
  if (wave < 4 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float4 o = red[wi * 64 + b * 32 + lane];
      const int ua2 = __float_as_int(o.z);
      sum[b] += o.x;
      if (o.y > amax[b] || (o.y == amax[b] && ua2 < uarg[b])) { amax[b] = o.y; uarg[b] = ua2; }
      p.partials[(int64_t)s * p.Np + rt * 256 + wi * 64 + b * 32 + lane] = make_float4(sum[b], amax[b] * p.sc, __int_as_float(uarg[b]), 0.f);
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

// single workgroup: n_valid, number of out-of-range targets, mean loss from the per-block sums (fixed order)
__global__ __launch_bounds__(1024) void fwd_reduce_kernel(const float4* __restrict__ partials, int nblk,
                                                         int32_t* __restrict__ hdr, float* __restrict__ loss_out,
                                                         int32_t* __restrict__ nvalid_out) {
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
  }
}

}  // namespace sce
