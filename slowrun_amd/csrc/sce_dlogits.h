// The block-scaled e4m3 format of the stored dlogits and the epilogue that forms it from a finished logit tile
// (shared by the forward kernel and the recompute kernel; internal header).
// Part of the one translation unit sce_kernels.hip, which includes it after the headers it builds on.
#pragma once

namespace sce {

// ------------------------------------------------------------------------------------------
// dlogits on chip
// ------------------------------------------------------------------------------------------
// The softmax part of dlogits, without the factors that belong to a whole row, is
//   D_iv = (1 - t^2) e^{z - cap} = 4 r (1 - r) e^{z - cap},  r = 1 / (1 + e^{2u/cap}),   0 <= D <= 1,
// and  du_iv = rho_i D_iv - (one-hot terms),  rho_i = g_i S_i e^{cap - lse_i}.  D is kept in e4m3 with one power-of-two
// exponent per block of 32 rows i x 128 columns v (MX style: byte * 2^(E - 127), E in an E8M0 byte), taken from the
// block's own largest logit, so that neither the row's final lse nor its maximum has to be known when the block is
// formed -- the forward pass can emit it -- and a peak in one place of a row costs the rest of the row nothing.  The
// dX and dW GEMMs apply the exponents inside the matrix instruction (mfma_mainloop, SCALE).
// Rows of very different temperature may share a block (a row whose logits saturate the cap next to ordinary ones:
// D near 0.05 next to D near e^{-cap}), and 8 bits cannot hold both at one exponent.  So each row also has a boost of
// its own, D_iv 2^{lam_i} is what is stored, with lam_i = -log2 Z_i, Z_i = sum_v e^{z_iv - cap} the row's softmax sum -- known
// when backward forms the dlogits (bwd_prep_kernel), estimated from two tiles of the row's logits and rounded down to an
// integer before a forward pass that emits them (fwd_sample_kernel) -- and undone in rho_i.  What is stored is then
// the row's probabilities, p_iv (1 - t^2) (times 2^f, 0 <= f < 1, for the integer), and rows that share a block are
// weighed by what their entries contribute.  The block exponent is taken after the boost, so a poor estimate costs
// precision, never range: an estimate of the sum that is too low boosts the row too far, and the 31 rows that share
// its blocks lose bits where its peaks are.
//
// Layout: G, tile by tile ([tile of 256 rows i][block of 128 columns v][256 i][128 v] bytes): the B operand of dX as it
// lies (rows i, K = v), and of dW (rows v, K = i) through the transposing LDS read.  Exponents: one dword per
// (128 v, 128 i), byte c for rows [32 c, 32 c + 32), as gexp[v / 128][i / 128].
//
// One wave turns its 128 (v) x 128 (i) quadrant of a finished logit tile into its quadrant of G and returns the dword
// of exponents of its four 32-row blocks.  A lane holds, of one row i, the columns 8 q + 4 h + (0..3) of every group of
// 32 (q = 0..3, h = its half-wave): the two lanes of a row swap two of their four words (v_permlane32_swap) and then
// hold 16 consecutive columns each, which go out as one 16-byte store.  No LDS is involved.
// STATS: the forward pass's row statistics as well (sum of e^{z - cap}, largest raw logit and its column), kept in
// `stat` (LDS, 12 floats per lane: [sum, max, argmax][4 row blocks], NTHREADS apart).

// Maximum over the 64 lanes, in every lane.  The lane exchanges are LDS-crossbar swizzles with the pattern in the
// instruction (xor 1 .. 16 within a half-wave), and one ds_bpermute across the halves whose address comes from
// lane_id(): __shfl_xor would keep its own copy of the lane index alive across the main loop, where it is spilled.
__device__ __forceinline__ float wave_max(float v) {
#define SCE_SWZ_MAX(X) v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), ((X) << 10) | 0x1f)))
  SCE_SWZ_MAX(1); SCE_SWZ_MAX(2); SCE_SWZ_MAX(4); SCE_SWZ_MAX(8); SCE_SWZ_MAX(16);
#undef SCE_SWZ_MAX
  return fmaxf(v, __int_as_float(__builtin_amdgcn_ds_bpermute((lane_id() ^ 32) << 2, __float_as_int(v))));
}

// The same without the LDS crossbar (whose operations queue behind the fragment reads of the other wave of the SIMD in
// the ping-pong kernel): four DPP steps leave the maximum of each row of 16 lanes in all of its lanes, the four rows
// meet through scalar registers.
__device__ __forceinline__ float wave_max_dpp(float v) {
#define SCE_DPP_MAX(CTRL) v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xF, 0xF, false)))
  SCE_DPP_MAX(0xB1);      // quad_perm [1, 0, 3, 2]
  SCE_DPP_MAX(0x4E);      // quad_perm [2, 3, 0, 1]
  SCE_DPP_MAX(0x141);     // row_half_mirror
  SCE_DPP_MAX(0x140);     // row_mirror
#undef SCE_DPP_MAX
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)), r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32)), r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// A tile that reaches beyond the vocabulary (columns >= vlim of the tile do not exist): their accumulators are set to
// -inf before the epilogue, which then needs no masking variant (two copies of it, each with the MFMAs that ride along,
// make the compiler spill accumulators) -- such a logit reads as z = -cap, its
// stored value is exactly 0, it cannot be a block's maximum, and what it adds to the row sum, e^{-2 cap} a piece, is
// taken out of `stat` here (a caller without row statistics passes none).  Row blocks [B0, B1).
template <int B0, int B1>
__device__ __forceinline__ void strike_columns_beyond(v16f (&acc)[4][4], int vlim, int wa, float* stat = nullptr, float em2cap = 0.f) {
  const int vloc0 = wa * 128 + 4 * (lane_id() >> 5);
  int cnt = 0;
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const bool out = vloc0 + a * 32 + 8 * (r >> 2) + (r & 3) >= vlim;
      cnt += out ? 1 : 0;
#pragma unroll
      for (int b = B0; b < B1; ++b) acc[a][b][r] = out ? -INFINITY : acc[a][b][r];
    }
  if (stat) {
#pragma unroll
    for (int b = B0; b < B1; ++b) stat[(0 + b) * NTHREADS] -= (float)cnt * em2cap;
  }
}

// lam (LDS, wave-uniform base; per row block LAM_STRIDE floats apart, one float for each of LAM_LANES lanes): the row's
// exponent boost (see fwd_sample_kernel).
// want_argmax (uniform, STATS only): see the lookup of the maximum's column below.
// gq: the wave's quadrant of G (128 rows i of 128 bytes, contiguous).
// B0, B1: the row blocks [B0, B1) only (the returned dword has their bytes).
// hook(b, k), k = 0..31: called between the stages of row block b's arithmetic (four to a batch of eight values): a place
// for a caller's matrix instructions on other accumulators.
// EXCL: the lane's values of row block b hold a target logit that is still in the accumulators (it has not been knocked
// out; its byte of G is cleared afterwards), known by its value: the accumulator times `sc` equals xc[b] (NaN: none).  It
// takes no part in the block's exponent -- the lane offers its second largest value when the largest is that one.
template <bool STATS, int LAM_STRIDE = NTHREADS, int LAM_LANES = 64, int B0 = 0, int B1 = 4, class Hook = NoHook, bool EXCL = false>
__device__ __forceinline__ uint32_t form_dlogits(const v16f (&acc)[4][4], float k1, float c2, int vabs0,
                                                 uint8_t* __restrict__ gq, int wa, int wb, float* stat, const float* lam, bool want_argmax = true,
                                                 Hook&& hook = NoHook(), const float* xc = nullptr, float sc = 0.f) {
  constexpr bool HOOKED = !std::is_same<typename std::decay<Hook>::type, NoHook>::value;
  uint32_t expword = 0;
#pragma unroll
  for (int b = B0; b < B1; ++b) {
    __builtin_amdgcn_sched_barrier(0);      // the next row block's accumulator reads stay behind this one's work: moved up, they do not fit the registers
    uint8_t* grow = gq + (b * 32 + (lane_id() & 31)) * BK + 16 * (lane_id() >> 5);      // the lane's row, its half of each 32 columns
    // the block's largest logit fixes its exponent: D * 2^s <= 2^(lg + s) <= 446 with lg = log2 e^{zmax - cap}
    float tmax = -INFINITY;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        tmax = fmaxf(tmax, acc[a][b][r]);
      }
    float texp = tmax, lfloor = -INFINITY;
    if (EXCL) {
      // some lane's largest value is its row's target (seldom, unless the rows are sure of their targets): that lane
      // offers the largest of the others
      const bool is_target = tmax * sc == xc[b];
      if (__builtin_amdgcn_ballot_w64(is_target) != 0) {
        // (a value that occurs twice among the lane's 64 is not the target alone -- all logits are equal under a head
        // that starts at zero -- and stays in: the other one needs the exponent)
        float tsec = -INFINITY;
        int ties = 0;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const bool same = acc[a][b][r] == tmax;
            ties += same ? 1 : 0;
            tsec = fmaxf(tsec, same ? -INFINITY : acc[a][b][r]);
          }
        if (is_target && ties == 1) {
          // (the exponent stays within 2^90 of the target all the same: the target's own e^{z - cap}, scaled like the rest,
          // still goes into the row sum, and must not leave the floats' range when everything else is at -cap under a large cap)
          texp = tsec;
          lfloor = c2 * fast_rcp(1.0f + fast_exp2(tmax * k1)) - 90.0f;
        }
      }
    }
    const float lamb = lam[b * LAM_STRIDE + (lane_id() & (LAM_LANES - 1))];      // (index taken anew: see lane_id)
    const float rexp = fast_rcp(1.0f + fast_exp2(texp * k1));
    const float lg = wave_max_dpp(EXCL ? fmaxf(c2 * rexp, lfloor) + lamb : fmaf(c2, rexp, lamb));      // over the block: log2 of the largest boosted e^{z - cap}
    const float sb = fminf(floorf(8.8f - lg), 126.f);         // from -112 (boost <= 120) to 8 + 2 cap log2(e) - boost, held to what the exponent byte has
    const float cs = sb + 2.0f + lamb;                        // the 4 of 4 r (1 - r) and the row's boost ride along
    expword |= (uint32_t)(127 - (int)sb) << (8 * b);
    float ssum = 0.f;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      // stage by stage over the 16 values of the block: the transcendental unit is pipelined, a chain
      // of dependent exp2 / rcp / exp2 on one value at a time is not (the scheduler would rebuild the
      // chains to save registers, hence the barriers)
      constexpr int NB = 8;        // values per batch: 4, 8 and 16 measure alike
      float rr[16], gg[16];
#pragma unroll
      for (int g0 = 0; g0 < 16; g0 += NB) {
#pragma unroll
        for (int m = g0; m < g0 + NB; ++m) rr[m] = fast_exp2(acc[a][b][m] * k1);
        __builtin_amdgcn_sched_barrier(0);
        if (HOOKED) { hook(b, 4 * (2 * a + g0 / NB)); __builtin_amdgcn_sched_barrier(0); }
#pragma unroll
        for (int m = g0; m < g0 + NB; ++m) rr[m] = fast_rcp(rr[m] + 1.0f);
        __builtin_amdgcn_sched_barrier(0);
        if (HOOKED) { hook(b, 4 * (2 * a + g0 / NB) + 1); __builtin_amdgcn_sched_barrier(0); }
#pragma unroll
        for (int m = g0; m < g0 + NB; ++m) gg[m] = fast_exp2(fmaf(c2, rr[m], cs));
        __builtin_amdgcn_sched_barrier(0);
        if (HOOKED) { hook(b, 4 * (2 * a + g0 / NB) + 2); __builtin_amdgcn_sched_barrier(0); }
        if (STATS) {
#pragma unroll
          for (int m = g0; m < g0 + NB; ++m) ssum += gg[m];
        }
#pragma unroll
        for (int m = g0; m < g0 + NB; ++m) gg[m] *= rr[m] - rr[m] * rr[m];
        __builtin_amdgcn_sched_barrier(0);
        if (HOOKED) { hook(b, 4 * (2 * a + g0 / NB) + 3); __builtin_amdgcn_sched_barrier(0); }
      }
      // words d[q] = columns 8 q + 4 h .. + 3 of this group of 32.  After the two swaps the lower half-wave holds
      // (d0, d0', d1, d1') = columns 0..15 and the upper one (d2, d2', d3, d3') = columns 16..31 (x' = the other lane's x).
      uint32_t d[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) d[q] = cvt4_e4m3(gg[4 * q], gg[4 * q + 1], gg[4 * q + 2], gg[4 * q + 3]);
      const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
      const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
      *reinterpret_cast<v4i*>(grow + a * 32) = (v4i){(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
    }
    if (STATS) {
      stat[(0 + b) * NTHREADS] += ssum * fast_exp2(-cs);
      const float amax = stat[(4 + b) * NTHREADS];
      // The column of the maximum is looked up only when a tile reaches a lane's running maximum (on a tie the lower
      // column wins: the running one may be a target of this very tile, which take_target_logits has put there) -- which
      // some lane of the 64 does in nearly every tile of a walk of a few dozen: a caller that does not ask for the argmax
      // is spared it.  (A flag at run time, not a template parameter: without the lookup in the code the register
      // allocation of the rest changes, and accumulators end up in scratch memory.)
      if (want_argmax && __builtin_amdgcn_ballot_w64(tmax >= amax && tmax != -INFINITY) != 0) {
        if (tmax >= amax) {
          int targ = 0x7fffffff;
#pragma unroll
          for (int a = 3; a >= 0; --a) {
#pragma unroll
            for (int r = 15; r >= 0; --r) {
              const int vo = a * 32 + 8 * (r >> 2) + (r & 3);
              if (acc[a][b][r] == tmax) targ = vo;   // descending scan: lowest column wins
            }
          }
          if (tmax > amax || (targ != 0x7fffffff && vabs0 + targ < __float_as_int(stat[(8 + b) * NTHREADS]))) {
            stat[(4 + b) * NTHREADS] = tmax;
            stat[(8 + b) * NTHREADS] = __int_as_float(vabs0 + targ);
          }
        }
      }
    }
  }
  return expword;
}

}  // namespace sce
