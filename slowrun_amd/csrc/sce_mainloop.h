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
#include <type_traits>

namespace sce {

// The schedule of one K block: what a wave issues in each of the block's 32 MFMA slots (64 clocks each) besides the
// MFMA itself.  Two kinds of work are placed:
//   * fragment reads, in units of half a fragment (one ds_read_b128, or two transposing 8-byte reads): r1 = the 16
//     units of this block's second sub-step, n0 = units of the next block's first sub-step (readable from the barrier
//     `b2` on, which publishes that block), c0 = what n0 left of this block's own first sub-step.  Units go in the order in
//     which the MFMAs need their fragments: A0, B0..B3, A1, A2, A3.
//   * the 16 direct-to-LDS loads of a block: ldEM = loads of the block after the next into this block's LDS slot -- from
//     b2 on, or earlier behind an extra barrier `b1_after` that tells that every wave has its last fragments of this
//     block; ldL = the rest of the next block's loads.  The wait that publishes a block comes at b2 of the block before.
// The four waves of a workgroup run in step and share the compute unit's one path from L2 (64 bytes a clock: 16 clocks
// for a wave's 1 KB load), so one load per wave and 64-clock MFMA slot already fills that path while it lasts.  Measured
// at N = 65536, d = 2560, V = 50304, all three big kernels alike: two loads to a slot -- all 16 early, behind the publishing
// barrier, or all late -- 5 to 10 % slower than schedule 0; reads spread one to a slot (1), loads spread over 22 slots behind
// an extra barrier (2), and mixtures of the two: within 0.5 % of schedule 0.  At the clock this part grants under fp8 MFMA
// load the loop is bound neither by where its LDS reads sit nor by the lead its loads have.
#ifndef SCE_SCHED
#define SCE_SCHED 0
#endif
struct KSched {
  signed char ldL[32], ldEM[32], r1[32], c0[32], n0[32];
  int b1_after, b2;
};
constexpr KSched KSCHEDS[] = {
    // 0: fragment reads two to a slot in the second half of each sub-step, loads behind the barrier in the middle of the second
    {{1, 1, 1, 1, 1, 1, 1, 1}, {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 1},
     {0, 0, 0, 0, 0, 0, 0, 0, 2, 2, 2, 2, 2, 2, 2, 2}, {0}, {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 2, 2, 2, 2, 2, 2, 2, 2}, -1, 24},
    // 1: one read unit to a slot almost everywhere, barrier at slot 22, loads 22..31 and 0..5
    {{1, 1, 1, 1, 1, 1}, {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1},
     {0, 0, 0, 0, 0, 0, 2, 2, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1}, {1, 1, 1, 1, 1, 1},
     {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1}, -1, 22},
    // 2: the reads of 0; an extra barrier after slot 17 lets six loads go out in slots 18..23, the slots with reads take a load every other time
    {{1, 1, 0, 1, 1, 0, 1, 1}, {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 0, 1, 0, 1, 0, 1, 0},
     {0, 0, 0, 0, 0, 0, 0, 0, 2, 2, 2, 2, 2, 2, 2, 2}, {0}, {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 2, 2, 2, 2, 2, 2, 2, 2}, 17, 24},
};
constexpr KSched KS = KSCHEDS[SCE_SCHED];
constexpr int ksum(const signed char (&a)[32], int n) { int t = 0; for (int i = 0; i < n; ++i) t += a[i]; return t; }
constexpr int LOADS_E = ksum(KS.ldEM, KS.b2), LOADS_EM = ksum(KS.ldEM, 32), UNITS_N0 = ksum(KS.n0, 32);
static_assert(LOADS_EM + ksum(KS.ldL, 32) == 16, "a K block is 16 loads per wave");
static_assert(ksum(KS.r1, 32) == 16 && UNITS_N0 + ksum(KS.c0, 32) == 16, "a sub-step is 16 read units");
static_assert(ksum(KS.n0, KS.b2) == 0, "the next block cannot be read before the barrier that publishes it");
static_assert(LOADS_E == 0 || (KS.b1_after >= 0 && ksum(KS.ldEM, KS.b1_after + 1) == 0), "loads before b2 need the extra barrier");
constexpr int AHEAD_LOADS = LOADS_EM;      // loads of K block 1 that a prefetch (or the prologue) puts in flight
constexpr int UNIT_FRAG[8] = {0, 4, 5, 6, 7, 1, 2, 3};      // fragment (0-3: A, 4-7: B) of the q-th pair of read units

// The compiler must not see these loads: it would serialise every later LDS read behind
// vmcnt(0).  Completion is tracked by hand with s_waitcnt vmcnt before the barrier that
// publishes the data.  LDS_CONST is an immediate, so that the only scalar work per load is the one
// addition that forms M0.  (The instruction's own offset field is of no use for stepping through
// K: the hardware adds it to the LDS address as well as to the memory address.)  M0 is written and consumed inside the
// one asm statement; it cannot be named as a clobber (the compiler treats it as reserved and says that a clobber of
// it is not honoured), so this relies on the compiler not keeping a value of its own in M0 across the statement --
// it loads M0 immediately before each instruction of its own that reads it.
template <int LDS_CONST>
__device__ __forceinline__ void lds_direct_16(uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
  asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
               ::"s"(lds_addr), "n"(LDS_CONST), "v"(voff), "s"(sbase) : "memory", "scc");
}

// Global -> LDS loads of one tile: per wave, 16 instructions per K block (8 for A, 8 for B).
//
// TRB = false: both operands are K-contiguous in memory (rows lda / ldb bytes apart) and in LDS.
// TRB = true : the B operand comes from an array that has the B rows (N) contiguous and K as the slow index,
//              stored in 128-byte pieces: for each of the 128 K rows of a K block, 128 bytes of N in one piece
//              and the next 128 bytes in a second piece `ldb` bytes further on.  In LDS the K block is
//              [2 pieces][128 K rows][128 B]; fragments are formed with the transposing LDS read (see below).
template <bool TRB = false>
struct TileLoads {
  uint32_t vo[16];    // per-lane byte offset of load n; even n: A, odd n: B
  uint32_t lds[16];   // LDS address of load n in slot 0 (wave-uniform)
  // load n of an operand covers the 8-row chunk (n / 2 + rot) % 8 of the wave's 64 rows
  // a_rows (LDS, or null): row r of the A tile is row a_rows[r] of the array at Ag instead of row r -- a gather; the
  // offsets stay 32-bit, so (largest index + 1) * lda must be below 2^32
  __device__ __forceinline__ TileLoads(int64_t lda, int64_t ldb, uint8_t* smem, int rot_a, int rot_b, int wave, const int* a_rows = nullptr) {
    const int lane = lane_id();
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    // one wave instruction covers 8 rows x 128 B; a wave fills rows [64 w, 64 w + 64) of A and of B
    const int lr = lane >> 3, pc = lane & 7;
#pragma unroll
    for (int n = 0; n < 8; ++n) {
      const int ca = (n + rot_a) & 7, cb = (n + rot_b) & 7;
      const int rowa = wave * 64 + ca * 8 + lr, rowb = wave * 64 + cb * 8 + lr;
      const int swa = (rowa & 7) ^ ((rowa >> 3) & 1), swb = (rowb & 7) ^ ((rowb >> 3) & 1);
      vo[2 * n] = (uint32_t)((a_rows ? a_rows[rowa] : rowa) * lda + ((pc ^ swa) * 16));
      if (TRB) vo[2 * n + 1] = (uint32_t)((rowb >> 7) * ldb + (rowb & 127) * BK + ((pc ^ (rowb & 7)) * 16));
      else vo[2 * n + 1] = (uint32_t)(rowb * ldb + ((pc ^ swb) * 16));
      lds[2 * n] = lds0 + wave * 64 * BK + ca * 8 * BK;
      lds[2 * n + 1] = lds0 + TM * BK + wave * 64 * BK + cb * 8 * BK;
    }
  }
  // load n of the K block that starts at ga / gb, into LDS slot SLOT
  template <int SLOT>
  __device__ __forceinline__ void issue(int n, const uint8_t* ga, const uint8_t* gb) const {
    lds_direct_16<SLOT * SLOT_BYTES>(lds[n], vo[n], (n & 1) ? gb : ga);
  }
};

// Puts K block 0 and the first AHEAD_LOADS loads of K block 1 of a tile in flight (16 + AHEAD_LOADS loads per wave).
// Both LDS slots must be free: every wave is past the closing barrier of the previous main loop.  A
// main loop that follows with PREFETCHED = true expects these loads to be the wave's newest
// vector memory loads, in this order (stores issued in between do not disturb the count it waits for:
// vector memory operations complete in order, so at most AHEAD_LOADS of them outstanding means block 0 has landed).
// PARTS: 1 = block 0 only (slot 0), 2 = the loads of block 1 only (slot 1), 3 = both.
template <int PARTS = 3>
__device__ __forceinline__ void mfma_prefetch(const uint8_t* __restrict__ Ag, int64_t lda, const uint8_t* __restrict__ Bg,
                                              int64_t ldb, uint8_t* smem, int rot_a, int rot_b, int wave) {
  const TileLoads<false> ld(lda, ldb, smem, rot_a, rot_b, wave);
  if (PARTS & 1) {
#pragma unroll
    for (int n = 0; n < 16; ++n) ld.issue<0>(n, Ag, Bg);
  }
  if (PARTS & 2) {
#pragma unroll
    for (int n = 0; n < AHEAD_LOADS; ++n) ld.issue<1>(n, Ag + BK, Bg + BK);
  }
}

// lda, ldb: row strides in bytes, multiples of 16, at most 2^24; KD = K / 128, even, >= 2;
// rot_a, rot_b in [0, 8), uniform over the workgroup; wave: index of the wavefront in the workgroup (scalar).
struct NoHook {
  __device__ __forceinline__ void operator()(int) const {}
  __device__ __forceinline__ void operator()(int, int) const {}
};

// `hook(i)` is called after MFMA i (0..63) of every pair of K blocks: a place for vector ALU work that
// does not depend on the accumulators (it runs while the matrix pipe is busy).
// TRB (see TileLoads): the K blocks of B lie bk1 bytes apart within a pair and bk2 bytes from pair to pair
// (for TRB = false they are KSTEP and 2 KSTEP and the two arguments are ignored).
//
// SCALE: the B operand is block-scaled (MX style): its true value is byte * 2^(E - 127) with one E8M0 exponent E per
// block of 32 B rows x 128 bytes of K or so, applied by v_mfma_scale_f32_32x32x64_f8f6f4 (lane l supplies, in the byte of
// its scale register that the instruction's op_sel names, the exponent of B row l % 32 for K values [0, 32) of the
// instruction if l < 32 and [32, 64) otherwise).
// The exponents of a tile wait in LDS behind the two K slots, one dword per K block for each half (wb) of the B rows:
//   SCALE = 1: byte b of the dword of K block k belongs to the wave's B rows [32 b, 32 b + 32) (dX: B = dlogits, K = v);
//   SCALE = 2: byte c of the dword of K block k belongs to K values [32 c, 32 c + 32) of that block, for all of the
//              wave's 128 B rows (dW: B = the columns of the dlogits, K = i, TRB).
// The A operand goes in with exponent 127 (factor 1).  lds_scale points at the wave's KD dwords.
template <int OPB>
__device__ __forceinline__ v16f mfma_fp8_scaled(const v8i& a, const v8i& b, const v16f& c, int sa, int sb) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, sa, OPB, sb);
}
__device__ __forceinline__ v16f mfma_fp8_scaled_sel(int opb, const v8i& a, const v8i& b, const v16f& c, int sa, int sb) {
  switch (opb) {       // op_sel is part of the instruction: the callers' loops are unrolled, so this folds
    case 0: return mfma_fp8_scaled<0>(a, b, c, sa, sb);
    case 1: return mfma_fp8_scaled<1>(a, b, c, sa, sb);
    case 2: return mfma_fp8_scaled<2>(a, b, c, sa, sb);
    default: return mfma_fp8_scaled<3>(a, b, c, sa, sb);
  }
}

// BF16: the operands are bf16 (64 K values per 128-byte block) and each step is two v_mfma_f32_32x32x16_bf16, on the
// first and the second 16 bytes of the lanes' fragments; everything else -- loads, LDS, the schedule in bytes -- is the same.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
__device__ __forceinline__ v16f mfma_bf16_pair(const v8i& a, const v8i& b, v16f c) {
  const v4i a0 = {a[0], a[1], a[2], a[3]}, a1 = {a[4], a[5], a[6], a[7]}, b0 = {b[0], b[1], b[2], b[3]}, b1 = {b[4], b[5], b[6], b[7]};
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a0), __builtin_bit_cast(v8bf, b0), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a1), __builtin_bit_cast(v8bf, b1), c, 0, 0, 0);
}

// DEFER (plain fp8 only): of the last pair of K blocks only the MFMAs of B block 0 (accumulators acc[.][0]) are
// issued; the other 48 are left to the caller, who finds the pair in the two LDS slots on return (lds_fragment) and
// issues them (mfma_tail) between the vector instructions of its epilogue of the finished accumulators, where the
// matrix pipe would otherwise stand idle.  Nothing may be loaded into the slots until that is done.
template <bool PREFETCHED = false, class Hook = NoHook, int KSTEP = BK, bool TRB = false, int SCALE = 0, bool BF16 = false, bool DEFER = false>
__device__ __forceinline__ void mfma_mainloop(const uint8_t* __restrict__ Ag, int64_t lda,
                                              const uint8_t* __restrict__ Bg, int64_t ldb, int KD,
                                              uint8_t* smem, v16f (&acc)[4][4], int rot_a, int rot_b, int wave, Hook&& hook = NoHook(),
                                              int64_t bk1_arg = 0, int64_t bk2_arg = 0, const uint32_t* lds_scale = nullptr,
                                              const int* a_rows = nullptr) {
  static_assert(!DEFER || (!BF16 && SCALE == 0 && !TRB), "DEFER is for the plain fp8 loop");
  const int lane = lane_id();
  const int wa = wave >> 1, wb = wave & 1;
  const int64_t bk1 = TRB ? bk1_arg : (int64_t)KSTEP, bk2 = TRB ? bk2_arg : (int64_t)(2 * KSTEP);
  const TileLoads<TRB> ld(lda, ldb, smem, rot_a, rot_b, wave, a_rows);
  // fragments: lane reads row l%32 of a 32-row block, 32 bytes of K at (l/32)*32 within the sub-step
  const int r = lane & 31, h = lane >> 5;
  const int sw = (r & 7) ^ ((r >> 3) & 1);
  const int abase = wa * 128 * BK + r * BK, bbase = TM * BK + wb * 128 * BK + r * BK;
  // half `u` (0, 1) of fragment n (0-3: A, 4-7: B) of the sub-step with K half `half` in LDS slot `slot`: registers 4 u .. 4 u + 3
  auto runit = [&](int slot, int half, int n, int u, v8i (&fa)[4], v8i (&fb)[4]) {
    v4i q;
    if (TRB && n >= 4) {
      // B block b = n - 4 from the [K row][N] layout.  ds_read_b64_tr_b8 works on groups of 16 lanes: lane j of a
      // group points at 8 bytes -- here the half (j & 1) of the 16-byte N chunk of K row (j >> 1) -- and gets byte j of
      // each of the group's 8 rows: 8 consecutive K values of its own N.  Four reads give the lane its 32 K values.
      // Group g = lane / 16 holds N chunk 2 b + (g & 1) and K half g / 2; the chunks of a row are XOR-swizzled by
      // (K row & 7) = j >> 1 (the loader stores them so).
      // Which 32 of the sub-step's 64 K rows a lane takes: registers 4 u .. 4 u + 3 hold rows 32 h + 16 u .. + 15, or, where the
      // exponent changes along K (SCALE = 2, see below), rows 32 u + 16 h .. + 15 -- the same choice as for the other operand.
      const int b = n - 4, g = lane >> 4, j = lane & 15;
      const int krow = 64 * half + (SCALE == 2 ? 32 * u + 16 * (g >> 1) : 32 * (g >> 1) + 16 * u) + (j >> 1);
      const uint8_t* s = smem + slot * SLOT_BYTES + TM * BK + wb * 128 * BK + krow * BK + (((2 * b + (g & 1)) ^ (j >> 1)) << 4) + 8 * (j & 1);
      const v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)(s));
      const v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)(s + 8 * BK));
      q = (v4i){r0[0], r0[1], r1[0], r1[1]};
    } else {
      // Which 32 of the sub-step's 64 K bytes a lane takes does not matter as long as both operands agree -- except
      // to the block scales: the instruction counts registers 0..3 of lanes l and l + 32 as the first 32 K values (scale
      // from lane l < 32) and registers 4..7 of both as the second 32 (scale from lane l + 32).  With per-K exponents
      // (SCALE = 2) the lanes therefore take the 16-byte chunks h and 2 + h, otherwise 2 h and 2 h + 1.
      const int c0 = ((SCALE == 2 ? 4 * half + h : 4 * half + 2 * h) ^ sw) * 16;
      const uint8_t* s = smem + slot * SLOT_BYTES + ((n < 4) ? abase + n * 32 * BK : bbase + (n - 4) * 32 * BK);
      q = *reinterpret_cast<const v4i*>(s + (u ? (c0 ^ (SCALE == 2 ? 32 : 16)) : c0));
    }
    v8i& f = n < 4 ? fa[n] : fb[n - 4];
    f[4 * u] = q[0]; f[4 * u + 1] = q[1]; f[4 * u + 2] = q[2]; f[4 * u + 3] = q[3];
  };
  // read units [q0, q0 + cnt) of a sub-step, in the order in which its MFMAs need them
  auto runits = [&](int slot, int half, int q0, int cnt, v8i (&fa)[4], v8i (&fb)[4]) {
#pragma unroll
    for (int q = q0; q < q0 + cnt; ++q) runit(slot, half, UNIT_FRAG[q >> 1], q & 1, fa, fb);
  };
  // prologue: K block 0 and half of block 1 in flight, block 0 visible, fragments of sub-step 0 in registers
  if (!PREFETCHED) {
#pragma unroll
    for (int n = 0; n < 16; ++n) ld.template issue<0>(n, Ag, Bg);
#pragma unroll
    for (int n = 0; n < AHEAD_LOADS; ++n) ld.template issue<1>(n, Ag + KSTEP, Bg + bk1);
  }
  // K block 0 has landed once at most the loads of block 1 are in flight (vector memory operations that a caller issued
  // after its prefetch -- stores of an epilogue -- are younger still: the wait then covers block 1 as well, no more)
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(AHEAD_LOADS) : "memory");
  v8i fa[2][4], fb[2][4];
  runits(0, 0, 0, 16, fa[0], fb[0]);
  // block scales of the current pair of K blocks and of the next one (read one pair ahead)
  const __attribute__((address_space(3))) v2i* scp = (const __attribute__((address_space(3))) v2i*)lds_scale;
  const int sc_shift = (SCALE == 2) ? 8 * (lane >> 5) : 0;      // SCALE = 2: the upper half-wave feeds the odd 32-blocks of K
  int sc[2] = {0, 0}, scn[2] = {0, 0};
  auto sc_load = [&](int (&dst)[2]) {
    const v2i d = *scp++;
    dst[0] = (int)((uint32_t)d[0] >> sc_shift); dst[1] = (int)((uint32_t)d[1] >> sc_shift);
  };
  if (SCALE) sc_load(sc);
  // blk: which K block of the pair; cur: fragment register set = which 64-byte half of the block
  auto mm = [&](int blk, int cur, int i) {
    const int a = i >> 2, b = i & 3;
    if (BF16) acc[a][b] = mfma_bf16_pair(fa[cur][a], fb[cur][b], acc[a][b]);
    else if (SCALE) acc[a][b] = mfma_fp8_scaled_sel(SCALE == 1 ? b : 2 * cur, fa[cur][a], fb[cur][b], acc[a][b], 127, sc[blk]);
    else acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[cur][a], fb[cur][b], acc[a][b], 0, 0, 0, 0, 0, 0);
  };
  // the very first MFMA of each accumulator block takes a zero constant instead of the register: nothing clears them
  auto mm0 = [&](int i) {
    const int a = i >> 2, b = i & 3;
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (BF16) acc[a][b] = mfma_bf16_pair(fa[0][a], fb[0][b], zero);
    else if (SCALE) acc[a][b] = mfma_fp8_scaled_sel(SCALE == 1 ? b : 0, fa[0][a], fb[0][b], zero, 127, sc[0]);
    else acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[0][a], fb[0][b], zero, 0, 0, 0, 0, 0, 0);
  };
  // One K block = two sub-steps of 16 MFMAs; register set 0 feeds the first, set 1 the second.  The loop body handles
  // the blocks in pairs (LDS slot 0, then slot 1) so that every LDS address and every load offset is a constant; what
  // goes into which MFMA slot is the table KS (above).  ga / gb point at the first block of the current pair; `more` tells
  // whether a further pair follows.
  const uint8_t* ga = Ag;
  const uint8_t* gb = Bg;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  // loads [n0, n0 + cnt) of the K block at pa / pb into LDS slot SLOT
  auto loads = [&](auto slot_tag, int n0, int cnt, const uint8_t* pa, const uint8_t* pb) {
#pragma unroll
    for (int n = n0; n < n0 + cnt; ++n) ld.template issue<decltype(slot_tag)::value>(n, pa, pb);
  };
  // block BLK (0, 1) of the pair, in LDS slot BLK.  p1a / p1b: the next block, p2a / p2b: the one after it; has1 / has2: they exist.
  auto block = [&](auto blk_tag, bool first, bool has1, bool has2, const uint8_t* p1a, const uint8_t* p1b, const uint8_t* p2a, const uint8_t* p2b) {
    constexpr int BLK = decltype(blk_tag)::value;
    using Own = std::integral_constant<int, BLK>;
    using Other = std::integral_constant<int, 1 - BLK>;
#pragma unroll
    for (int s = 0; s < 32; ++s) {
      if (s == KS.b2) {
        // every wave has all fragments of this block in registers (its reads are complete, not only issued) and its own
        // loads of the next block have landed: the barrier frees this block's LDS slot and publishes the next block
        if (has1) {
          if (has2) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(LOADS_E) : "memory");
          else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      const int sub = s >> 4, i = s & 15;
      if (DEFER && !has2 && (i & 3) != 0) {}      // last pair, B blocks 1 - 3: the caller's
      else if (first && BLK == 0 && sub == 0) mm0(i); else mm(BLK, sub, i);
      hook(32 * BLK + s);
      if (!(first && BLK == 0)) runits(BLK, 0, UNITS_N0 + ksum(KS.c0, s), KS.c0[s], fa[0], fb[0]);      // (the first block's came with the prologue)
      runits(BLK, 1, ksum(KS.r1, s), KS.r1[s], fa[1], fb[1]);
      if (has1) {
        runits(1 - BLK, 0, ksum(KS.n0, s), KS.n0[s], fa[0], fb[0]);
        loads(Other(), LOADS_EM + ksum(KS.ldL, s), KS.ldL[s], p1a, p1b);
      }
      if (has2) loads(Own(), ksum(KS.ldEM, s), KS.ldEM[s], p2a, p2b);
      __builtin_amdgcn_sched_barrier(0);
      if (s == KS.b1_after && has2) {
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  auto pair = [&](bool first, bool more) {
    block(I0(), first, true, more, ga + KSTEP, gb + bk1, ga + 2 * KSTEP, gb + bk2);
    if (SCALE && more) sc_load(scn);
    block(I1(), false, more, more, ga + 2 * KSTEP, gb + bk2, ga + 3 * KSTEP, gb + bk2 + bk1);
    if (SCALE && more) { sc[0] = scn[0]; sc[1] = scn[1]; }
  };
  const int P = KD >> 1;
  if (P == 1) {
    if (DEFER) {       // the only pair is the last one: what it leaves undone starts from zero
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 1; b < 4; ++b)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
    }
    pair(true, false);
  } else {
    pair(true, true);
    ga += 2 * KSTEP;
    gb += bk2;
    for (int p = 1; p < P - 1; ++p) {
      pair(false, true);
      ga += 2 * KSTEP;
      gb += bk2;
    }
    pair(false, false);
  }
  // all LDS reads of this tile are complete in every wave before the caller reuses the buffer
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Reader of the fragments of the pair of K blocks in the two LDS slots, as the plain fp8 main loop reads them; the lane's
// part of the addresses is computed once (lb[half][u]: the lane's row and the swizzled 16-byte chunks 2 h + u of the
// 64-byte half `half` of a K block).
struct TailReader {
  const uint8_t* lb[2][2];
  int wa, wb;
  __device__ __forceinline__ TailReader(const uint8_t* smem, int wa_, int wb_) : wa(wa_), wb(wb_) {
    const int lane = lane_id(), r = lane & 31, h = lane >> 5, sw = (r & 7) ^ ((r >> 3) & 1);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int c0 = ((4 * half + 2 * h) ^ sw) * 16;
      lb[half][0] = smem + r * BK + c0; lb[half][1] = smem + r * BK + (c0 ^ 16);
    }
  }
  // fragment n (0 - 3: A block n, 4 - 7: B block n - 4) of sub-step `step` (0 - 3: K block step / 2, its half step % 2)
  __device__ __forceinline__ v8i operator()(int step, int n) const {
    const int off = (step >> 1) * SLOT_BYTES + (n < 4 ? wa * 128 * BK + n * 32 * BK : TM * BK + wb * 128 * BK + (n - 4) * 32 * BK);
    const v4i q0 = *reinterpret_cast<const v4i*>(lb[step & 1][0] + off), q1 = *reinterpret_cast<const v4i*>(lb[step & 1][1] + off);
    return (v8i){q0[0], q0[1], q0[2], q0[3], q1[0], q1[1], q1[2], q1[3]};
  }
};
// The 48 MFMAs that a DEFER main loop has left undone, handed out one call at a time: a caller's epilogue of row block
// 0 calls (acc, 0, k), k = 0..31, between the stages of its arithmetic and gets the 32 MFMAs of row blocks 1 and 2, one a
// call; its epilogue of row block 1 calls (acc, 1, k), k = 0..31, and gets the 16 of row block 3 at every other call.
// After that the LDS slots are free.  Every fragment is read two calls before its first use, into registers that the
// MFMAs in between do not use: the A fragments alternate between fa[0] and fa[1], the B fragments of a sub-step between
// fb[0] and fb[1].
//
// What a call does is a table, tail_op(b, k), that the device code follows and that tail_schedule_ok() replays at
// compile time: every one of the 48 (sub-step, A block, row block) products is issued exactly once, in ascending
// sub-step order for each accumulator block (the order the main loop itself would have used), from registers that
// hold the right fragments, each read at least two calls earlier.
struct TailRead { int kind, i, j, step, n; };       // register (kind 0: fa[i]; kind 1: fb[i][j]) <- fragment n of sub-step `step`
struct TailOp {
  bool mfma;                                         // acc[a][rb] += fa[fa_i] x fb[fb_i][fb_j] (sub-step `step`)
  int step, a, rb, fa_i, fb_i, fb_j;
  int nreads;
  TailRead reads[3];
};
constexpr int TAIL_CALLS = 32;                       // calls per row block epilogue (8 batches of 4 stages)
constexpr TailOp tail_prologue() {                   // before the first call
  return TailOp{false, 0, 0, 0, 0, 0, 0, 3, {{0, 0, 0, 0, 0}, {1, 0, 0, 0, 5}, {1, 0, 1, 0, 6}}};
}
constexpr TailOp tail_op(int b, int k) {
  TailOp op{false, 0, 0, 0, 0, 0, 0, 0, {{0, 0, 0, 0, 0}, {0, 0, 0, 0, 0}, {0, 0, 0, 0, 0}}};
  if (b == 0) {
    // MFMA k of 32: sub-step k / 8, A block (k % 8) / 2, row block 1 + k % 2
    const int s = k >> 3, a = (k & 7) >> 1;
    op.mfma = true; op.step = s; op.a = a; op.rb = 1 + (k & 1); op.fa_i = a & 1; op.fb_i = s & 1; op.fb_j = k & 1;
    const int k2 = k + 2, s2 = k2 >> 3, a2 = (k2 & 7) >> 1;       // what MFMA k + 2 needs
    if (k2 < 32) {
      if ((k2 & 1) == 0) op.reads[op.nreads++] = TailRead{0, a2 & 1, 0, s2, a2};
      if ((k2 & 7) == 0) {
        op.reads[op.nreads++] = TailRead{1, s2 & 1, 0, s2, 5};
        op.reads[op.nreads++] = TailRead{1, s2 & 1, 1, s2, 6};
      }
    } else if (k2 == 32) {                                        // the first of row block 3's
      op.reads[op.nreads++] = TailRead{0, 0, 0, 0, 0};
      op.reads[op.nreads++] = TailRead{1, 0, 0, 0, 7};
    }
  } else if (b == 1 && (k & 1)) {
    // MFMA m = k / 2 of 16: sub-step m / 4, A block m % 4, row block 3
    const int m = k >> 1, s = m >> 2, a = m & 3;
    op.mfma = true; op.step = s; op.a = a; op.rb = 3; op.fa_i = a & 1; op.fb_i = s & 1; op.fb_j = 0;
    const int m2 = m + 1, s2 = m2 >> 2, a2 = m2 & 3;
    if (m2 < 16) {
      op.reads[op.nreads++] = TailRead{0, a2 & 1, 0, s2, a2};
      if (a2 == 0) op.reads[op.nreads++] = TailRead{1, s2 & 1, 0, s2, 7};
    }
  }
  return op;
}
constexpr bool tail_schedule_ok() {
  int fa_frag[2] = {-1, -1}, fa_when[2] = {0, 0};            // which fragment (8 * step + n) a register holds, and since which call
  int fb_frag[2][2] = {{-1, -1}, {-1, -1}}, fb_when[2][2] = {{0, 0}, {0, 0}};
  int done[4][4][4] = {};                                     // [step][a][rb]
  int next_step[4][4] = {};                                   // [a][rb]: the sub-step this accumulator block expects next
  int call = 0;
  auto apply = [&](const TailOp& op) {
    for (int q = 0; q < op.nreads; ++q) {
      const TailRead& r = op.reads[q];
      if (r.kind == 0) { fa_frag[r.i] = 8 * r.step + r.n; fa_when[r.i] = call; }
      else { fb_frag[r.i][r.j] = 8 * r.step + r.n; fb_when[r.i][r.j] = call; }
    }
  };
  apply(tail_prologue());
  call = 2;                                                   // the prologue's reads have had the time before the first call
  for (int b = 0; b < 2; ++b)
    for (int k = 0; k < TAIL_CALLS; ++k, ++call) {
      const TailOp op = tail_op(b, k);
      if (op.mfma) {
        if (fa_frag[op.fa_i] != 8 * op.step + op.a || fb_frag[op.fb_i][op.fb_j] != 8 * op.step + 4 + op.rb) return false;
        if (call - fa_when[op.fa_i] < 2 || call - fb_when[op.fb_i][op.fb_j] < 2) return false;
        if (next_step[op.a][op.rb] != op.step) return false;
        ++next_step[op.a][op.rb];
        ++done[op.step][op.a][op.rb];
      }
      apply(op);
    }
  for (int s = 0; s < 4; ++s)
    for (int a = 0; a < 4; ++a)
      for (int rb = 1; rb < 4; ++rb)
        if (done[s][a][rb] != 1) return false;
  return true;
}
static_assert(tail_schedule_ok(), "the deferred MFMAs: some product missing, doubled, out of order, or fed from the wrong registers");

struct DeferredTail {
  TailReader frag;
  v8i fa[2], fb[2][2];
  __device__ __forceinline__ void read(const TailOp& op) {
#pragma unroll
    for (int q = 0; q < 3; ++q)
      if (q < op.nreads) {
        const TailRead& r = op.reads[q];
        if (r.kind == 0) fa[r.i] = frag(r.step, r.n); else fb[r.i][r.j] = frag(r.step, r.n);
      }
  }
  __device__ __forceinline__ DeferredTail(const uint8_t* smem, int wa, int wb) : frag(smem, wa, wb) { read(tail_prologue()); }
  __device__ __forceinline__ void operator()(v16f (&acc)[4][4], int b, int k) {
    const TailOp op = tail_op(b, k);
    if (op.mfma) acc[op.a][op.rb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[op.fa_i], fb[op.fb_i][op.fb_j], acc[op.a][op.rb], 0, 0, 0, 0, 0, 0);
    read(op);
  }
};

}  // namespace sce
