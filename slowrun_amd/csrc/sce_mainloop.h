// MFMA main loop shared by the forward, recompute, dX and dW kernels (internal header).
//
// acc[a][b] (32x32 blocks) = A_tile[256][K] * B_tile[256][K]^T in fp8 e4m3 on
// v_mfma_f32_32x32x64_f8f6f4.  Wave (wa, wb) of the 2 x 2 wave grid owns A rows [128 wa, +128)
// and B rows [128 wb, +128).
//
// Data path: global memory -> LDS directly (global_load_lds_dwordx4, no staging registers), in
// full 128-byte row segments (half-line requests ran at about half the L2 bandwidth per CU).
// Two 64 KB LDS slots each hold K = 128 bytes of the 512 tile rows.  16-byte chunks are XOR
// swizzled by row so that fragment reads are free of bank conflicts without padding (a wave-wide
// direct load fills 1 KB of LDS contiguously, so padding rows is not possible).  Fragments are
// double-buffered in registers one 64-byte sub-step ahead; there is one barrier per K block,
// placed in the middle of its second sub-step, and the instruction order (one MFMA, then its
// share of LDS reads and global loads) is pinned with sched_barrier.
//
// Workgroups that run side by side on one XCD share tile rows through its L2.  Each of them
// starts its loads of a K block at a different 8-row chunk (rot_a, rot_b: the workgroup's index
// among the sharers of its A and B rows), so that together they touch every line of the block
// at the start of the issue window: whichever line misses L2 is requested as early as possible,
// and the others find it there (measured +7 to +13 % on operands that come from HBM).
#pragma once
#include "sce_common.h"

namespace sce {

// The compiler must not see these loads: it would serialise every later LDS read behind
// vmcnt(0).  Completion is tracked by hand with s_waitcnt vmcnt before the barrier that
// publishes the data.
__device__ __forceinline__ void lds_direct_16(uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}

// lda, ldb: row strides in bytes, multiples of 16, at most 2^24; KD = K / 128 >= 2;
// rot_a, rot_b in [0, 8), uniform over the workgroup.
__device__ __forceinline__ void mfma_mainloop(const uint8_t* __restrict__ Ag, int64_t lda,
                                              const uint8_t* __restrict__ Bg, int64_t ldb, int KD,
                                              uint8_t* smem, v16f (&acc)[4][4], int rot_a, int rot_b) {
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6), wa = wave >> 1, wb = wave & 1;
  const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
  // global -> LDS: one wave instruction covers 8 rows x 128 B; a wave fills rows [64 w, 64 w + 64) of A and of B
  const int lr = lane >> 3, pc = lane & 7;
  uint32_t vo[16];   // even: A, odd: B; load n of an operand covers the 8-row chunk (n + rot) % 8
#pragma unroll
  for (int n = 0; n < 8; ++n) {
    const int rowa = wave * 64 + ((n + rot_a) & 7) * 8 + lr, rowb = wave * 64 + ((n + rot_b) & 7) * 8 + lr;
    const int swa = (rowa & 7) ^ ((rowa >> 3) & 1), swb = (rowb & 7) ^ ((rowb >> 3) & 1);
    vo[2 * n] = (uint32_t)(rowa * lda + ((pc ^ swa) * 16));
    vo[2 * n + 1] = (uint32_t)(rowb * ldb + ((pc ^ swb) * 16));
  }
  auto issue1 = [&](int kd, int n) {
    const int chunk = ((n >> 1) + ((n & 1) ? rot_b : rot_a)) & 7;
    const uint32_t base = lds0 + (kd & 1) * SLOT_BYTES + (n & 1) * TM * BK + wave * 64 * BK + chunk * 8 * BK;
    const uint8_t* g = ((n & 1) ? Bg : Ag) + (int64_t)kd * BK;
    lds_direct_16(base, vo[n], g);
  };
  // fragments: lane reads row l%32 of a 32-row block, 32 bytes of K at (l/32)*32 within the sub-step
  const int r = lane & 31, h = lane >> 5;
  const int sw = (r & 7) ^ ((r >> 3) & 1);
  const int abase = wa * 128 * BK + r * BK, bbase = TM * BK + wb * 128 * BK + r * BK;
  auto rfrag1 = [&](int j, int n, v8i (&fa)[4], v8i (&fb)[4]) {   // sub-step j, fragment n (0-3: A, 4-7: B)
    const int c0 = ((4 * (j & 1) + 2 * h) ^ sw) * 16;
    const uint8_t* s = smem + ((j >> 1) & 1) * SLOT_BYTES + ((n < 4) ? abase + n * 32 * BK : bbase + (n - 4) * 32 * BK);
    const v4i lo = *reinterpret_cast<const v4i*>(s + c0);
    const v4i hi = *reinterpret_cast<const v4i*>(s + (c0 ^ 16));
    const v8i f = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (n < 4) fa[n] = f; else fb[n - 4] = f;
  };
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[a][b][q] = 0.f;

  // prologue: K blocks 0 and 1 in flight, block 0 visible, fragments of sub-step 0 in registers
#pragma unroll
  for (int n = 0; n < 16; ++n) issue1(0, n);
#pragma unroll
  for (int n = 0; n < 16; ++n) issue1(1, n);
  asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory");
  v8i fa[2][4], fb[2][4];
#pragma unroll
  for (int n = 0; n < 8; ++n) rfrag1(0, n, fa[0], fb[0]);
  auto mm = [&](int cur, int i) {
    const int a = i >> 2, b = i & 3;
    acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[cur][a], fb[cur][b], acc[a][b], 0, 0, 0, 0, 0, 0);
  };
  const int J = 2 * KD;
  // Sub-step j works from register set `cur`.  After the barrier of an odd sub-step every wave has
  // its fragments of K block (j-1)/2 in registers, so that slot is refilled with block (j+3)/2:
  // 8 loads in the second half of this sub-step, 8 in the first half of the next.  The barrier of
  // the next odd sub-step waits for them (vmcnt(0)) and publishes the block.
  auto substep = [&](int j, int cur, bool odd) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mm(cur, i);
      if (!odd && j > 0 && ((j + 2) >> 1) < KD) issue1((j + 2) >> 1, 8 + i);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (odd && j + 1 < J) asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    const int kd_new = (j + 3) >> 1;
#pragma unroll
    for (int i = 8; i < 16; ++i) {
      mm(cur, i);
      if (j + 1 < J) rfrag1(j + 1, i - 8, fa[cur ^ 1], fb[cur ^ 1]);
      if (odd && kd_new < KD) issue1(kd_new, i - 8);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  for (int j = 0; j < J; j += 2) {
    substep(j, 0, false);
    substep(j + 1, 1, true);
  }
  // all LDS reads of this tile are complete in every wave before the caller reuses the buffer
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

}  // namespace sce
