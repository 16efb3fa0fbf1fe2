// Device kernels of the measurement aids (sce_bench_mfma, sce_bench_gemm): the matrix instruction alone, the main loop
// alone (internal header).
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

// The main loops of the three big kernels alone, on the very buffers a forward and backward call have filled, in their
// own layouts and tile orders: what fwd_kernel, bwd_dx_kernel and bwd_dw_kernel would take with an epilogue of nothing
// (each thread stores the sum of its accumulators at the end).  The difference to the real kernels is their epilogues,
// the difference to the peak is the main loop's.
__device__ __forceinline__ float acc_sum(const v16f (&acc)[4][4]) {
  float sum = 0.f;
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[a][b][r];
  return sum;
}
__device__ __forceinline__ void floor_clock(long long* clk, long long c0, long long r0) {
  if (threadIdx.x == 0 && blockIdx.x < 1024) {
    clk[2 * blockIdx.x] = __builtin_readcyclecounter() - c0; clk[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

// the walk of fwd_kernel (one workgroup: a row tile and its share of the column tiles, next tile prefetched), no epilogue
__global__ __launch_bounds__(256) void floor_fwd_kernel(FwdParams p, float* __restrict__ out, long long* __restrict__ clk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int rt, s;
  if (!map_tile(blockIdx.x, p.RT, p.S, rt, s)) return;
  const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  const int ct0 = (int)((int64_t)p.CT * s / p.S), ct1 = (int)((int64_t)p.CT * (s + 1) / p.S);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  v16f acc[4][4];
  const uint8_t* Bg = p.xq + (int64_t)rt * 256 * p.ldx;
  const int KT = (int)(p.dp / BK);
  const int rot_a = 2 * (rt & 3), rot_b = s & 7;
  float sum = 0.f;
  if (ct0 < ct1) mfma_prefetch(p.wqt + (int64_t)ct0 * 256 * p.ldx, p.ldx, Bg, p.ldx, smem, rot_a, rot_b, wave);
  for (int ct = ct0; ct < ct1; ++ct) {
    mfma_mainloop<true>(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, Bg, p.ldx, KT, smem, acc, rot_a, rot_b, wave);
    if (ct + 1 < ct1) mfma_prefetch(p.wqt + (int64_t)(ct + 1) * 256 * p.ldx, p.ldx, Bg, p.ldx, smem, rot_a, rot_b, wave);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) sum += acc[a][b][0];      // (one value of each block keeps its MFMAs alive)
  }
  out[(int64_t)blockIdx.x * 256 + threadIdx.x] = sum;
  floor_clock(clk, c0, r0);
}

__global__ __launch_bounds__(256) void floor_dx_kernel(DxParams p, float* __restrict__ out, long long* __restrict__ clk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int rt, ct;
  if (!map_tile(blockIdx.x, p.RT, p.CT, rt, ct)) return;
  const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  const int KD = (int)(p.Vp / BK);
  const int t = threadIdx.x, wave = t >> 6, wb = wave & 1;
  uint32_t* lsc = reinterpret_cast<uint32_t*>(smem + SMEM_BYTES);
  for (int e = t; e < 2 * KD; e += NTHREADS) {
    const int w = e >= KD, kb = e - w * KD;
    lsc[e] = p.gexp[(int64_t)kb * p.kbw + 2 * rt + w];
  }
  __syncthreads();
  v16f acc[4][4];
  mfma_mainloop<false, NoHook, BLOCKED_KSTEP, false, 1>(p.wq + (int64_t)ct * (p.Vp / BK) * BLOCKED_KSTEP, BK,
                                                        p.ghat_t + (int64_t)rt * (p.Vp / BK) * BLOCKED_KSTEP, BK, KD, smem, acc,
                                                        2 * (rt & 3), ct & 7, __builtin_amdgcn_readfirstlane(wave), NoHook(), 0, 0,
                                                        lsc + __builtin_amdgcn_readfirstlane(wb) * KD);
  out[(int64_t)blockIdx.x * 256 + threadIdx.x] = acc_sum(acc);
  floor_clock(clk, c0, r0);
}

__global__ __launch_bounds__(256) void floor_dw_kernel(DwParams p, float* __restrict__ out, long long* __restrict__ clk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  int rt, ct;
  if (!map_tile_rr(blockIdx.x, p.RT, p.CT, rt, ct)) return;
  const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  const int t = threadIdx.x, wave = t >> 6, wb = wave & 1;
  uint32_t* lsc = reinterpret_cast<uint32_t*>(smem + SMEM_BYTES);
  for (int e = t; e < 2 * p.KT; e += NTHREADS) {
    const int w = e >= p.KT, kb = e - w * p.KT;
    lsc[e] = p.gexp[(int64_t)(2 * ct + w) * p.kbw + kb];
  }
  __syncthreads();
  v16f acc[4][4];
  mfma_mainloop<false, NoHook, BLOCKED_KSTEP, true, 2>(p.xt + ((int64_t)rt * p.kbn + p.kb0) * BLOCKED_KSTEP, BK, p.ghat_t + (int64_t)(2 * ct) * BLOCKED_KSTEP, BLOCKED_KSTEP, p.KT,
                                                       smem, acc, ct & 7, 2 * (rt & 3), __builtin_amdgcn_readfirstlane(wave), NoHook(), 128 * BK, p.kbv * BLOCKED_KSTEP,
                                                       lsc + __builtin_amdgcn_readfirstlane(wb) * p.KT);
  out[(int64_t)blockIdx.x * 256 + threadIdx.x] = acc_sum(acc);
  floor_clock(clk, c0, r0);
}

}  // namespace sce
