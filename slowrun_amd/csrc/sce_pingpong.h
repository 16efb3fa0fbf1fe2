// Ping-pong walk over logit tiles: the matrix pipe and the vector ALU of a SIMD work at the same time, on different
// tiles (internal header).
//
// A workgroup of 8 wavefronts (two per SIMD) walks T column half-tiles -- 128 rows of the A-side operand (W_q^T) each --
// of one 256-row tile of the B-side operand (X_q).  Waves 0-3 are group 0, waves 4-7 group 1; a SIMD holds one wave of
// each.  Tile j is accumulated by group j & 1 (each wave a 128 x 64 piece: 128 accumulator registers) while the other
// group runs the epilogue of tile j - 1 on the accumulators it finished a moment ago: one group issues MFMAs, the other
// transcendentals and conversions, and the hardware interleaves the two instruction streams.  With one wave per SIMD
// and a 256 x 256 tile the epilogue has nothing to hide behind (a finished tile fills the register file).
//
// The price is operand traffic: a 256 x 128 tile moves 1.5 times the bytes per flop of a 256 x 256 one through L2 and
// LDS, which is what bounds the walk when K is long; it wins where the epilogue is a large share of the tile time.
//
// LDS ring: three stages of 48 KB, each one K block (128 bytes of K) of the 256 B-side rows and of the 128 A-side rows
// of the tile that is being accumulated; blocks of consecutive tiles follow each other without a gap.  Step n consumes
// block n.  Every step has exactly one workgroup barrier, B_n, in both roles.  After B_n nobody reads the stage of
// block n any more, and block n + 3 is loaded into it (global_load_lds_dwordx4, 48 instructions of 8 rows x 128 B per
// block, shared out among the waves: LK per wave of the accumulating group, 12 - LK per wave of the other); every wave
// waits for its own loads of block n + 1 before it arrives at B_n, so that block has landed for everybody after it.
//
// The epilogue is handed over as Epi::UNITS pieces of straight-line code, Epi::unit(u, acc, j), which the walk spreads
// over the K steps of the other group's tile (units [k U / KD, (k + 1) U / KD) in step k).
#pragma once
#include "sce_mainloop.h"

namespace sce {

constexpr int PP_THREADS = 512;
constexpr int PP_STAGE = 48 * 1024;
constexpr int PP_RING = 3 * PP_STAGE;        // 147456

__device__ __forceinline__ void lds_direct_16_rt(uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}

// Xg: the 256 B-side rows (row stride ld); Wg: row 0 of the first half-tile of the A side (same stride; the half-tiles
// follow each other, 128 rows apart); KD = K / 128, even, >= 2; T >= 1; smem: PP_RING bytes; wave in [0, 8), scalar.
// acc[a][b] of wave (g, wi): A rows [32 a, +32) of the half-tile, B rows [64 wi + 32 b, +32).
template <class Epi, int LK>
__device__ __forceinline__ void pingpong_walk(const uint8_t* __restrict__ Xg, const uint8_t* __restrict__ Wg, int64_t ld, int KD, int T,
                                              uint8_t* smem, int wave, Epi& epi) {
  static_assert(LK == 0 || LK == 6 || LK == 12, "shares the wait counts know");
  const int lane = lane_id();
  const int grp = wave >> 2, wi = wave & 3;
  const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
  // ---- loads.  Instruction idx of a block (0..31: B-side rows [8 idx, +8); 32..47: A-side rows [8 (idx - 32), +8)) lands
  // at stage + idx * 1024; 8 lanes cover the 128 bytes of a row, 16-byte chunks XOR-swizzled by row as the fragment
  // reads expect ((row & 7) ^ ((row >> 3) & 1): the second term is the parity of idx).
  uint32_t vo2[2];
  {
    const int lr = lane >> 3, pc = lane & 7;
    vo2[0] = (uint32_t)(lr * ld + ((pc ^ lr) * 16));
    vo2[1] = (uint32_t)(lr * ld + ((pc ^ lr ^ 1) * 16));
  }
  const int total = T * KD;
  int ml = 0, kl = 0;                 // next block to load and its K index
  const uint8_t* gx = Xg;
  const uint8_t* gw = Wg;
  const int64_t ld8 = 8 * ld;
  // (Every lambda below is always_inline: one that is left as a call takes what it captures -- the accumulators, the
  // fragments, the epilogue's state -- out of the registers and into scratch memory.)
  // A wave of the accumulating group issues LKX of the 32 B-side instructions of a block and LKW of the 16 A-side ones,
  // a wave of the other group the rest of its quarter (all counts even, so that the parity of an instruction's index,
  // which its swizzle depends on, is known at compile time).
  constexpr int LKX = LK * 2 / 3, LKW = LK / 3, LEX = 8 - LKX, LEW = 4 - LKW;
  const int ikx = wi * LKX, ikw = wi * LKW, iex = 4 * LKX + wi * LEX, iew = 4 * LKW + wi * LEW;    // first instruction of the wave's shares
  // load t of this wave's share of block ml (krole: the wave belongs to the accumulating group)
  auto issue_one = [&](uint32_t soff, bool krole, int t) __attribute__((always_inline)) {
    if (ml < total) {
      const int nx = krole ? LKX : LEX;
      if (t < nx) {
        const int idx = (krole ? ikx : iex) + t;
        lds_direct_16_rt(lds0 + soff + idx * 1024, vo2[t & 1], gx + idx * ld8);
      } else {
        const int idx = (krole ? ikw : iew) + (t - nx);
        lds_direct_16_rt(lds0 + soff + 32 * 1024 + idx * 1024, vo2[(t - nx) & 1], gw + idx * ld8);
      }
    }
  };
  auto advance_loads = [&]() __attribute__((always_inline)) {
    ++ml; ++kl; gx += BK; gw += BK;
    if (kl == KD) { kl = 0; gx = Xg; gw += 128 * ld - (int64_t)KD * BK; }
  };
  // Before B_n: the wave's loads of block n + 1 have landed; its loads of block n + 2, issued in the previous step in
  // the role it had then, may still be in flight (vector memory operations complete in order; stores that an epilogue
  // unit issued in between only make the wait stricter).
  auto wait_block = [&](int n, bool krole_prev) __attribute__((always_inline)) {
    const int cnt = (n + 2 < total) ? (krole_prev ? LK : 12 - LK) : 0;
    if (cnt >= 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else if (cnt >= 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (cnt >= 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else if (cnt >= 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  // ---- fragments: lane reads row l % 32 of a 32-row block, 32 bytes of K at (l / 32) * 32 within the 64-byte sub-step
  const int r = lane & 31, h = lane >> 5;
  const int sw = (r & 7) ^ ((r >> 3) & 1);
  const int abase = 32 * 1024 + r * BK, bbase = wi * 64 * BK + r * BK;
  // A fragments are single-buffered: fragment a of the next sub-step is read as soon as the two MFMAs that use the
  // current one have been issued (six MFMAs ahead of its first use); B fragments are double-buffered.
  v8i fa[4], fb[2][2];
  auto rfrag_a = [&](uint32_t soff, int half, int a) __attribute__((always_inline)) {
    const int c0 = ((4 * half + 2 * h) ^ sw) * 16;
    const uint8_t* s = smem + soff + abase + a * 32 * BK;
    const v4i lo = *reinterpret_cast<const v4i*>(s + c0);
    const v4i hi = *reinterpret_cast<const v4i*>(s + (c0 ^ 16));
    fa[a] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto rfrag_b = [&](uint32_t soff, int half, int b, v8i (&dst)[2]) {
    const int c0 = ((4 * half + 2 * h) ^ sw) * 16;
    const uint8_t* s = smem + soff + bbase + b * 32 * BK;
    const v4i lo = *reinterpret_cast<const v4i*>(s + c0);
    const v4i hi = *reinterpret_cast<const v4i*>(s + (c0 ^ 16));
    dst[b] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  v16f acc[4][2];
  uint32_t cur = 0, nxt = PP_STAGE;      // stages of block n and of block n + 1
  auto rotate = [&]() __attribute__((always_inline)) { cur = nxt; nxt = (nxt + PP_STAGE == PP_RING) ? 0u : nxt + PP_STAGE; };
  int n = 0;
  // One K step of the accumulating group: 16 MFMAs, m = 8 sub + 2 a + b, on the two 64-byte halves (sub-steps) of block
  // n.  The fragments of sub-step 0 are in registers when the step begins.  B_n stands after the first pair of sub-step
  // 1: by then every fragment of block n has been requested, and the ones requested last have had two MFMAs to arrive.
  // After it come the first fragments of block n + 1 (more: this group goes on with it) and the wave's share of block n + 3.
  auto kstep = [&](bool first, bool more, bool krole_prev) __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int sub = m >> 3, a = (m >> 1) & 3, b = m & 1;
      if (first && sub == 0) {        // the first MFMA of a tile takes a zero constant: nothing clears the accumulators
        const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[a], fb[0][b], zero, 0, 0, 0, 0, 0, 0);
      } else {
        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[a], fb[sub][b], acc[a][b], 0, 0, 0, 0, 0, 0);
      }
      if (m == 9) {
        __builtin_amdgcn_sched_barrier(0);
        wait_block(n, krole_prev);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
      if (b == 1) {
        if (sub == 0) rfrag_a(cur, 1, a);
        else if (more) rfrag_a(nxt, 0, a);
      }
      if (sub == 0 && (m == 2 || m == 4)) rfrag_b(cur, 1, (m - 2) >> 1, fb[1]);
      if (sub == 1 && more && (m == 10 || m == 12)) rfrag_b(nxt, 0, (m - 10) >> 1, fb[0]);
      if (m >= 10) {
#pragma unroll
        for (int t = 0; t < LK; ++t)
          if (t % 6 == m - 10) issue_one(cur, true, t);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    advance_loads(); rotate(); ++n;
  };
  // the first fragments of a tile, for the group that starts on it after the next barrier
  auto first_frags = [&](uint32_t soff) __attribute__((always_inline)) {
#pragma unroll
    for (int a = 0; a < 4; ++a) rfrag_a(soff, 0, a);
#pragma unroll
    for (int b = 0; b < 2; ++b) rfrag_b(soff, 0, b, fb[0]);
  };
  // prologue: every wave requests 6 instructions of each of the first three blocks
  for (int q = 0; q < 3; ++q) {
    if (ml < total) {
#pragma unroll
      for (int t = 0; t < 6; ++t) {
        const int idx = wave * 6 + t;
        const uint8_t* src = idx < 32 ? gx + idx * ld8 : gw + (idx - 32) * ld8;
        lds_direct_16_rt(lds0 + q * PP_STAGE + idx * 1024, (idx & 1) ? vo2[1] : vo2[0], src);
      }
    }
    advance_loads();
  }
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  if (grp == 0) first_frags(0);
  // Round j: group j & 1 accumulates tile j, the other group runs the epilogue of tile j - 1 (there is none in round 0).
  // In round T only an epilogue is left; the group without one keeps the barriers company.
  for (int j = 0; j <= T; ++j) {
    // The compiler knows nothing of the tile loads (inline asm), so any wait of its own on the vector memory counter --
    // for a register it reloads from scratch memory at a change of role, say -- also waits for every tile load in flight.
    // Such a wait inside the loops of steps would serialise the walk; this one, once per tile, tells the compiler that
    // nothing of its own is pending when the loops begin.
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    if (grp == (j & 1) && j < T) {
#ifndef PP_NOPRIO
      __builtin_amdgcn_s_setprio(3);       // the accumulating wave issues first whenever it can: the matrix pipe is the scarcer one
#endif
      kstep(true, true, false);
      for (int k = 1; k < KD - 1; ++k) kstep(false, true, true);
      kstep(false, false, true);
    } else {
      const bool have = j >= 1 && grp != (j & 1);
#ifndef PP_NOPRIO
      __builtin_amdgcn_s_setprio(0);
#endif
      epi.begin();
      int u = 0, ucarry = 0;      // units [k U / KD, (k + 1) U / KD) in step k, without the divisions
      for (int k = 0; k < KD; ++k) {
        ucarry += Epi::UNITS;
        if (have) {
          for (; ucarry >= KD; ucarry -= KD, ++u) epi.unit(u, acc, j - 1);
        }
        wait_block(n, k == 0);
        asm volatile("s_barrier" ::: "memory");
#pragma unroll
        for (int t = 0; t < 12 - LK; ++t) issue_one(cur, false, t);
        advance_loads(); rotate(); ++n;
      }
      // the first fragments of the tile this group starts on next: its block 0 has landed and is published by the
      // barrier just passed
      if (j + 1 < T) first_frags(cur);
    }
  }
}

}  // namespace sce
