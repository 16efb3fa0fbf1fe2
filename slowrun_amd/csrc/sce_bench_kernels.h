// Device kernels of the measurement aids (sce_bench_mfma, sce_bench_gemm, sce_bench_pingpong): the matrix instruction
// alone, the main loop alone, the ping-pong walk with a synthetic epilogue (internal header).
// Part of the one translation unit sce_kernels.hip, which includes it after the headers it builds on.
#pragma once

namespace sce {

// ------------------------------------------------------------------------------------------
// measurement aids (sce_bench_*): what the matrix pipe and the main loop reach on their own
// ------------------------------------------------------------------------------------------
// The matrix instruction alone: every wave issues `iters` rounds of 16 independent v_mfma_f32_32x32x64_f8f6f4 on
// operands it keeps in registers (bytes from `data`, or a constant when data is NULL); no memory traffic in the loop.
// clk[2 w], clk[2 w + 1]: shader clocks and 100 MHz ticks that workgroup w's first wave spent in the loop.
__global__ __launch_bounds__(256) void bench_mfma_kernel(const uint8_t* __restrict__ data, int iters, float* __restrict__ out,
                                                        long long* __restrict__ clk) {
  v8i fa[4], fb[4];
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    if (data) {
      fa[n] = *reinterpret_cast<const v8i*>(data + ((size_t)(blockIdx.x * 256 + threadIdx.x) * 8 + n) * 32);
      fb[n] = *reinterpret_cast<const v8i*>(data + ((size_t)(blockIdx.x * 256 + threadIdx.x) * 8 + 4 + n) * 32);
    } else {
      fa[n] = (v8i){0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838};
      fb[n] = fa[n];
    }
  }
  v16f acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[a], fb[b], acc[a][b], 0, 0, 0, 0, 0, 0);
  }
  const long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float sum = 0.f;
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[a][b][r];
  out[blockIdx.x * 256 + threadIdx.x] = sum;
  if (threadIdx.x == 0 && blockIdx.x < 1024) { clk[2 * blockIdx.x] = c1 - c0; clk[2 * blockIdx.x + 1] = r1 - r0; }
}

// The main loop alone: C = A B^T over 256 x 256 tiles, both operands e4m3 rows of ld bytes; every thread writes the
// sum of its accumulators (so that the work cannot be dropped), nothing else.
__global__ __launch_bounds__(256) void bench_gemm_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ C,
                                                        int KD, int RT, int CT, int64_t ld, long long* __restrict__ clk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int rt, ct;
  if (!map_tile(blockIdx.x, RT, CT, rt, ct)) return;
  const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  v16f acc[4][4];
  mfma_mainloop(A + (int64_t)rt * 256 * ld, ld, B + (int64_t)ct * 256 * ld, ld, KD, smem, acc, ct & 7, 2 * (rt & 3),
                __builtin_amdgcn_readfirstlane(threadIdx.x >> 6));
  float sum = 0.f;
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[a][b][r];
  C[(int64_t)blockIdx.x * 256 + threadIdx.x] = sum;
  if (threadIdx.x == 0 && blockIdx.x < 1024) {
    clk[2 * blockIdx.x] = __builtin_readcyclecounter() - c0; clk[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

// The ping-pong walk (sce_pingpong.h) with a synthetic epilogue: COPIES times the transcendental and conversion work of
// the dlogits epilogue on every value (nothing stored but a checksum), or with COPIES = 0 only a sum of the
// accumulators.  Tells what the walk's operand traffic costs and how much of the vector ALU work of one wave of a SIMD
// is hidden behind the MFMAs of the other.
template <int COPIES>
struct BenchPPEpi {
  static constexpr int UNITS = 16;
  float s[2];
  uint32_t x;
  float k1, c2, cs;
  __device__ __forceinline__ void begin() {}
  template <int U>
  __device__ __forceinline__ void unit_c(const v16f (&acc)[4][2]) {
    constexpr int a = U >> 2, b = (U >> 1) & 1, g0 = (U & 1) * 8;
    if (COPIES == 0) {
#pragma unroll
      for (int m = 0; m < 8; ++m) s[b] += acc[a][b][g0 + m];
      return;
    }
    for (int rep = 0; rep < COPIES; ++rep) {
      float rr[8], gg[8];
      float k = k1;
      asm volatile("" : "+v"(k));      // (keeps the unit where it is called: see FwdPPEpi::values8)
#pragma unroll
      for (int m = 0; m < 8; ++m) rr[m] = fast_exp2(acc[a][b][g0 + m] * k);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < 8; ++m) rr[m] = fast_rcp(rr[m] + 1.0f);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < 8; ++m) gg[m] = fast_exp2(fmaf(c2, rr[m], cs));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < 8; ++m) s[b] += gg[m];
#pragma unroll
      for (int m = 0; m < 8; ++m) gg[m] *= rr[m] - rr[m] * rr[m];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const uint32_t w = cvt4_e4m3(gg[4 * q], gg[4 * q + 1], gg[4 * q + 2], gg[4 * q + 3]);
        const uint32_t p1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0xB1, 0xF, 0xF, true);
        const uint32_t xx = __builtin_amdgcn_perm(p1, w, 0x06020400u);
        const uint32_t p2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)xx, 0x4E, 0xF, 0xF, true);
        x ^= __builtin_amdgcn_perm(p2, xx, 0x05040100u);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __device__ __forceinline__ void unit(int u, const v16f (&acc)[4][2], int) {
    switch (u) {
#define SCE_BPP_CASE(U) case U: unit_c<U>(acc); break;
      SCE_BPP_CASE(0) SCE_BPP_CASE(1) SCE_BPP_CASE(2) SCE_BPP_CASE(3) SCE_BPP_CASE(4) SCE_BPP_CASE(5) SCE_BPP_CASE(6) SCE_BPP_CASE(7)
      SCE_BPP_CASE(8) SCE_BPP_CASE(9) SCE_BPP_CASE(10) SCE_BPP_CASE(11) SCE_BPP_CASE(12) SCE_BPP_CASE(13) SCE_BPP_CASE(14) SCE_BPP_CASE(15)
#undef SCE_BPP_CASE
      default: break;
    }
  }
};
// A: (M, K) rows that the walk takes 128 at a time; B: (N, K) rows in tiles of 256; every workgroup walks an eighth of A's half-tiles
template <int COPIES>
__global__ __launch_bounds__(PP_THREADS) void bench_pp_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ C,
                                                             int KD, int RT, int CT2, int64_t ld) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int rt, s;
  if (!map_tile(blockIdx.x, RT, 8, rt, s)) return;
  const int h0 = (int)((int64_t)CT2 * s / 8), h1 = (int)((int64_t)CT2 * (s + 1) / 8);
  BenchPPEpi<COPIES> e;
  e.s[0] = e.s[1] = 0.f; e.x = 0; e.k1 = 0.01f; e.c2 = -43.f; e.cs = 3.f;
  pingpong_walk<BenchPPEpi<COPIES>, 12>(B + (int64_t)rt * 256 * ld, A + (int64_t)h0 * 128 * ld, ld, KD, h1 - h0, smem,
                                        __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), e);
  C[(int64_t)blockIdx.x * PP_THREADS + threadIdx.x] = e.s[0] + e.s[1] + __uint_as_float(e.x & 0x3fffffff);
}

}  // namespace sce
