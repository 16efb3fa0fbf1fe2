// gfx950 (MI355X, CDNA4) kernels for the fused fp8 LM-head + tanh-softcap + cross-entropy
// loss head, and the C ABI declared in include/slowrun_ce.h.
//
// Replaces, in the reference: the quantise / _scaled_mm / ce_fwd_bwd / transpose_copy chain of
// FusedSoftcappedCrossEntropy (tiny/cuda_kernels.py:336-414, kernel at :125-302).
//
// Data flow
//   forward : X, W --quantise--> X_q [Np][dp], W_q^T [Vp][dp], W_q [dq][Vp]   (OCP e4m3, zero padded)
//             fwd_kernel: 256x256 logit tiles on v_mfma_f32_32x32x64_f8f6f4; the epilogue keeps per-row
//             sum exp(z - cap), the target logits and (on request) max/argmax of u; the logits never leave
//             the chip.  With dlogits_from_forward it also leaves D = (1 - t^2) exp(z - cap) as e4m3 bytes
//             with one power-of-two exponent per 32 rows x 128 columns (G^T, tile by tile), the targets'
//             entries zero.  Partials per (row, V-split) -> combine.  (fwd_pp_kernel: the same from 256x128
//             tiles with two waves per SIMD; opt-in.)
//   backward: the dlogits as forward left them, or formed again panel by panel from recomputed logit tiles
//             (bwd_recompute_kernel, same format); dX = rho_row * D W_q^T and dW = (rho X_q)^T D run on the
//             same MFMA main loop with the exponents applied inside v_mfma_scale_f32_32x32x64_f8f6f4.  The
//             one-hot part of dlogits never goes through fp8: it is applied in fp32 in the dX epilogue
//             (gather of W_q^T rows) and in the dW finalisation (rows grouped by target).
#include "sce_common.h"
#include "sce_mainloop.h"
#include "sce_pingpong.h"
#include "../../include/slowrun_ce.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <mutex>
#include <type_traits>
#include <vector>

namespace sce {

// ------------------------------------------------------------------------------------------
// small device helpers
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ float bf16_bits_to_float(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {   // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);   // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_float(float_to_bf16_bits(f)); }

// two floats -> two e4m3 bytes (low half of the result).  v_cvt_pk_fp8_f32 on gfx950 is OCP
// e4m3fn, round to nearest even, 464 -> 448 and anything larger -> NaN code: the same rule as
// Tensor.to(torch.float8_e4m3fn).
__device__ __forceinline__ uint32_t cvt2_e4m3(float a, float b) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}
__device__ __forceinline__ uint32_t cvt4_e4m3(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return (uint32_t)w;
}
template <int SEL>
__device__ __forceinline__ float e4m3_to_float(uint32_t word) { return __builtin_amdgcn_cvt_f32_fp8((int)word, SEL); }

template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  // x.div(s) with a host scalar s as torch's GPU kernels compute it: x * (1 / s), the reciprocal taken once in fp32
  // (the CPU kernels divide; the two differ in the last bit now and then, which moves an fp8 tie)
  static __device__ __forceinline__ float div_round(float x, float inv_s) { return x * inv_s; }
  // x.div(s) with s a device scalar (a 0-dim tensor): a true division, on the GPU too
  static __device__ __forceinline__ float div_true(float x, float s) { return x / s; }
};
struct bf16_t { uint16_t bits; };
template <> struct Elem<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_bits_to_float(p->bits); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }
  // torch scales a bf16 tensor in fp32 and rounds the result back to bf16 before the fp8 cast
  static __device__ __forceinline__ float div_round(float x, float inv_s) { return round_to_bf16(x * inv_s); }
  static __device__ __forceinline__ float div_true(float x, float s) { return round_to_bf16(x / s); }
};

// How the quantisers apply the fp8 scale: `by` is 1 / s (host scalar: multiplied in) or, with `divide`, s itself read
// from device memory (true division), in both cases what torch's GPU kernels do for that kind of divisor.
struct Scaler {
  float by;
  bool divide;
  template <typename T>
  __device__ __forceinline__ float apply(float x) const { return divide ? Elem<T>::div_true(x, by) : Elem<T>::div_round(x, by); }
};
// scale_dev != NULL: the scale lives on the device.  torch brings a 0-dim tensor divisor to the dtype of the tensor it
// divides before it divides (a bf16 tensor is divided by the scale rounded to bf16); a Python-float divisor is not.
template <typename T>
__device__ __forceinline__ Scaler make_scaler(float inv_host, const float* scale_dev) {
  Scaler sc;
  sc.divide = scale_dev != nullptr;
  sc.by = sc.divide ? (sizeof(T) == 2 ? round_to_bf16(*scale_dev) : *scale_dev) : inv_host;
  return sc;
}

// Scale-derived constants when a scale lives on the device (sce_args.x_s_dev / w_s_dev): written by dev_consts_kernel
// into the header of the saved state, read by every kernel that needs them in place of its by-value copies.
struct DevConsts {
  float x_s, w_s, sc, k1;      // sc = x_s w_s; k1 = sc 2 log2(e) / cap
};
__global__ void dev_consts_kernel(const float* xs_dev, const float* ws_dev, float xs_host, float ws_host, float cap, DevConsts* out) {
  DevConsts c;
  c.x_s = xs_dev ? *xs_dev : xs_host;
  c.w_s = ws_dev ? *ws_dev : ws_host;
  c.sc = c.x_s * c.w_s;
  c.k1 = c.sc * 2.0f * LOG2E / cap;
  *out = c;
}

// XCD-aware tile order.  Consecutive workgroup ids go round-robin to the 8 XCDs, each with its
// own L2.  The tiles are put in a locality-preserving order (groups of 8 columns, walked row by
// row, so that 32 consecutive tiles form a 4 x 8 block sharing A-side and B-side rows) and every
// XCD takes one contiguous eighth of that order: equal shares, and neighbours in the order run on
// the same L2 at about the same time.
__device__ __forceinline__ void tile_from_index(int idx, int RT, int CT, int& rt, int& ct) {
  const int gsz = 8 * RT;                 // tiles in a full group of 8 columns
  const int g = idx / gsz, rem = idx - g * gsz;
  const int gw = (CT - g * 8) < 8 ? (CT - g * 8) : 8;
  rt = rem / gw;
  ct = g * 8 + (rem - rt * gw);
}
__device__ __forceinline__ bool map_tile(int bid, int RT, int CT, int& rt, int& ct) {
  const int T = RT * CT;
  const int per = (T + 7) >> 3;
  const int xcd = bid & 7, local = bid >> 3;
  if (local >= per) return false;
  const int idx = xcd * per + local;
  if (idx >= T) return false;
  tile_from_index(idx, RT, CT, rt, ct);
  return true;
}
static inline int map_tile_grid(int RT, int CT) { return 8 * ((RT * CT + 7) / 8); }

// The same order, dealt out differently: blocks of 32 consecutive tiles go round-robin to the XCDs, so that the
// 256 workgroups that run at one time work on 256 consecutive tiles of the order (8 neighbouring 4 x 8 blocks).
// What the XCDs stream from memory at one time is then the same few operand tiles, not eight distant sets.
__device__ __forceinline__ bool map_tile_rr(int bid, int RT, int CT, int& rt, int& ct) {
  const int T = RT * CT;
  const int xcd = bid & 7, local = bid >> 3;
  const int idx = (((local >> 5) << 3) + xcd) * 32 + (local & 31);
  if (idx >= T) return false;
  tile_from_index(idx, RT, CT, rt, ct);
  return true;
}
static inline int map_tile_rr_grid(int RT, int CT) { return 256 * ((RT * CT + 255) / 256); }

// ------------------------------------------------------------------------------------------
// quantisation
// ------------------------------------------------------------------------------------------
// 16 consecutive elements starting at p as floats after the scaling; elements at or beyond
// `valid` are 0.  One or two 16/32-byte vector loads when the run is complete and 16-byte aligned.
template <typename T>
__device__ __forceinline__ void load16_scaled(const T* __restrict__ p, int64_t valid, const Scaler scale, float (&v)[16]) {
  if (valid >= 16 && (((uintptr_t)p) & 15) == 0) {
    if constexpr (sizeof(T) == 2) {
      const v4i r0 = *reinterpret_cast<const v4i*>(p), r1 = *reinterpret_cast<const v4i*>(p + 8);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        v[2 * m] = scale.apply<T>(__uint_as_float((uint32_t)r0[m] << 16));
        v[2 * m + 1] = scale.apply<T>(__uint_as_float((uint32_t)r0[m] & 0xffff0000u));
        v[8 + 2 * m] = scale.apply<T>(__uint_as_float((uint32_t)r1[m] << 16));
        v[8 + 2 * m + 1] = scale.apply<T>(__uint_as_float((uint32_t)r1[m] & 0xffff0000u));
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4f r = *reinterpret_cast<const v4f*>(p + 4 * q);
#pragma unroll
        for (int m = 0; m < 4; ++m) v[4 * q + m] = scale.apply<T>(r[m]);
      }
    }
  } else {
#pragma unroll
    for (int m = 0; m < 16; ++m) v[m] = (m < valid) ? scale.apply<T>(Elem<T>::load(p + m)) : 0.f;
  }
}

// dst [rows_p][cols_p] e4m3 = src [rows][cols] / s, zero outside; 16 outputs per thread.  In all the quantising
// kernels inv_scale is the reciprocal 1 / s taken once on the host, or, with scale_dev, s is read from the device.
template <typename T>
__global__ __launch_bounds__(256) void quantize_pad_kernel(const T* __restrict__ src, int64_t ld, int64_t rows,
                                                          int64_t cols, uint8_t* __restrict__ dst,
                                                          int64_t rows_p, int64_t cols_p, int64_t dst_ld, float inv_scale,
                                                          const float* __restrict__ scale_dev) {
  const Scaler scale = make_scaler<T>(inv_scale, scale_dev);
  const int64_t chunks_per_row = cols_p / 16;
  const int64_t total = rows_p * chunks_per_row;
  for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < total; q += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = q / chunks_per_row, c0 = (q - r * chunks_per_row) * 16;
    uint32_t out[4] = {0, 0, 0, 0};
    if (r < rows && c0 < cols) {
      float v[16];
      load16_scaled<T>(src + r * ld + c0, cols - c0, scale, v);
#pragma unroll
      for (int m = 0; m < 4; ++m) out[m] = cvt4_e4m3(v[4 * m], v[4 * m + 1], v[4 * m + 2], v[4 * m + 3]);
    }
    *reinterpret_cast<v4i*>(dst + r * dst_ld + c0) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
  }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// The trunk's last operation fused into the quantiser (F.rms_norm without weight, tiny/train.py:397-398,734):
// dst row = e4m3(round_T(h * rstd) / scale) with rstd = 1 / sqrt(mean(h^2) + eps), the normalised row rounded to
// the input's type as the unfused path has it in memory.  One wave per row; rstd is kept for backward.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_quantize_kernel(const T* __restrict__ src, int64_t ld, int64_t rows,
                                                              int64_t cols, float eps, uint8_t* __restrict__ dst,
                                                              int64_t rows_p, int64_t cols_p, int64_t dst_ld, float inv_scale,
                                                              const float* __restrict__ scale_dev, float* __restrict__ rstd_out) {
  const Scaler scale = make_scaler<T>(inv_scale, scale_dev), one = {1.0f, false};
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows_p) return;
  const int64_t chunks = cols_p / 16;
  if (r >= rows) {
    for (int64_t c = lane; c < chunks; c += 64) *reinterpret_cast<v4i*>(dst + r * dst_ld + c * 16) = (v4i){0, 0, 0, 0};
    if (lane == 0) rstd_out[r] = 0.f;
    return;
  }
  const T* row = src + r * ld;
  float ss = 0.f;
  for (int64_t c = lane; c * 16 < cols; c += 64) {
    float v[16];
    load16_scaled<T>(row + c * 16, cols - c * 16, one, v);      // scaling by 1 is exact: the values themselves
#pragma unroll
    for (int m = 0; m < 16; ++m) ss = fmaf(v[m], v[m], ss);
  }
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)cols + eps);
  if (lane == 0) rstd_out[r] = rstd;
  for (int64_t c = lane; c < chunks; c += 64) {
    uint32_t out[4] = {0, 0, 0, 0};
    if (c * 16 < cols) {
      float v[16];
      load16_scaled<T>(row + c * 16, cols - c * 16, one, v);
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        float y = v[m] * rstd;
        if constexpr (sizeof(T) == 2) y = round_to_bf16(y);
        v[m] = scale.apply<T>(y);
      }
#pragma unroll
      for (int m = 0; m < 4; ++m) out[m] = cvt4_e4m3(v[4 * m], v[4 * m + 1], v[4 * m + 2], v[4 * m + 3]);
    }
    *reinterpret_cast<v4i*>(dst + r * dst_ld + c * 16) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
  }
}

// 8 consecutive elements as floats, and back; `vec`: the run is 16-byte (bf16) / 32-byte (fp32) aligned.
template <typename T>
__device__ __forceinline__ void load8(const T* __restrict__ p, bool vec, float (&v)[8]) {
  if (vec) {
    if constexpr (sizeof(T) == 2) {
      const v4i r = *reinterpret_cast<const v4i*>(p);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        v[2 * m] = __uint_as_float((uint32_t)r[m] << 16);
        v[2 * m + 1] = __uint_as_float((uint32_t)r[m] & 0xffff0000u);
      }
    } else {
      const v4f a = *reinterpret_cast<const v4f*>(p), b = *reinterpret_cast<const v4f*>(p + 4);
#pragma unroll
      for (int m = 0; m < 4; ++m) { v[m] = a[m]; v[4 + m] = b[m]; }
    }
  } else {
#pragma unroll
    for (int m = 0; m < 8; ++m) v[m] = Elem<T>::load(p + m);
  }
}
template <typename T>
__device__ __forceinline__ void store8(T* __restrict__ p, bool vec, const float (&v)[8]) {
  if (vec) {
    if constexpr (sizeof(T) == 2) {
      v4i r;
#pragma unroll
      for (int m = 0; m < 4; ++m) r[m] = (int)((uint32_t)float_to_bf16_bits(v[2 * m]) | ((uint32_t)float_to_bf16_bits(v[2 * m + 1]) << 16));
      *reinterpret_cast<v4i*>(p) = r;
    } else {
      *reinterpret_cast<v4f*>(p) = (v4f){v[0], v[1], v[2], v[3]};
      *reinterpret_cast<v4f*>(p + 4) = (v4f){v[4], v[5], v[6], v[7]};
    }
  } else {
#pragma unroll
    for (int m = 0; m < 8; ++m) Elem<T>::store(p + m, v[m]);
  }
}

// Backward of that norm, in place on the finished dX: with xhat = h * rstd and g the gradient of the normalised row,
// dh = rstd * (g - xhat * mean(g * xhat)).  One wave per row; cols is a multiple of 8.
template <typename TG, typename TH>
__global__ __launch_bounds__(256) void rmsnorm_backward_kernel(TG* __restrict__ g, int64_t g_ld, const TH* __restrict__ h,
                                                              int64_t h_ld, const float* __restrict__ rstd_in, int64_t rows,
                                                              int64_t cols) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const float rstd = rstd_in[r];
  TG* grow = g + r * g_ld;
  const TH* hrow = h + r * h_ld;
  const bool gvec = (((uintptr_t)grow) & (8 * sizeof(TG) - 1)) == 0, hvec = (((uintptr_t)hrow) & (8 * sizeof(TH) - 1)) == 0;
  float dot = 0.f;
  for (int64_t c = 8 * lane; c < cols; c += 512) {
    float gv[8], hv[8];
    load8<TG>(grow + c, gvec, gv);
    load8<TH>(hrow + c, hvec, hv);
#pragma unroll
    for (int m = 0; m < 8; ++m) dot = fmaf(gv[m], hv[m] * rstd, dot);
  }
  dot = wave_sum(dot) / (float)cols;
  for (int64_t c = 8 * lane; c < cols; c += 512) {
    float gv[8], hv[8];
    load8<TG>(grow + c, gvec, gv);
    load8<TH>(hrow + c, hvec, hv);
#pragma unroll
    for (int m = 0; m < 8; ++m) gv[m] = rstd * (gv[m] - hv[m] * rstd * dot);
    store8<TG>(grow + c, gvec, gv);
  }
}

// Operands with a long K (the two of dW, and W_q in dX) are stored tile by tile: for every 256 rows, K block
// after K block, 256 rows of 128 bytes each.  A workgroup's load of one K block of one operand is then one
// contiguous 32 KB piece (row-major rows lie Np, Pw or Vp bytes apart, and the dW main loop lost 12 % to that at
// K = 65536).
__device__ __forceinline__ int64_t blocked_offset(int64_t row, int64_t k, int64_t kblocks) {
  return (((row >> 8) * kblocks + (k >> 7)) * 256 + (row & 255)) * 128 + (k & 127);
}
constexpr int BLOCKED_KSTEP = 256 * BK;     // bytes from one K block of a tile to the next

// W (d, V) -> W_q (dq rows, K = Vp, tile by tile) and W_q^T [Vp][dp] (row-major); 64 x 64 tiles through LDS.
template <typename T>
__global__ __launch_bounds__(256) void quantize_w_kernel(const T* __restrict__ w, int64_t ld, int64_t d, int64_t V,
                                                        uint8_t* __restrict__ wq, uint8_t* __restrict__ wqt,
                                                        int64_t dp, int64_t ldx, int64_t kbv, float inv_scale,
                                                        const float* __restrict__ scale_dev) {
  const Scaler scale = make_scaler<T>(inv_scale, scale_dev);
  __shared__ uint8_t tile[64][68];
  const int t = threadIdx.x;
  const int64_t j0 = (int64_t)blockIdx.y * 64, v0 = (int64_t)blockIdx.x * 64;
  {
    const int r = t >> 2, c = (t & 3) * 16;
    const int64_t j = j0 + r, v = v0 + c;
    uint32_t out[4] = {0, 0, 0, 0};
    if (j < d && v < V) {
      float x[16];
      load16_scaled<T>(w + j * ld + v, V - v, scale, x);
#pragma unroll
      for (int m = 0; m < 4; ++m) out[m] = cvt4_e4m3(x[4 * m], x[4 * m + 1], x[4 * m + 2], x[4 * m + 3]);
    }
    *reinterpret_cast<v4i*>(wq + blocked_offset(j, v, kbv)) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
#pragma unroll
    for (int m = 0; m < 4; ++m) *reinterpret_cast<uint32_t*>(&tile[r][c + 4 * m]) = out[m];
  }
  __syncthreads();
  if (j0 < dp) {
    const int vr = t >> 2, jc = (t & 3) * 16;
    uint32_t out[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      out[m] = (uint32_t)tile[jc + 4 * m][vr] | ((uint32_t)tile[jc + 4 * m + 1][vr] << 8) |
               ((uint32_t)tile[jc + 4 * m + 2][vr] << 16) | ((uint32_t)tile[jc + 4 * m + 3][vr] << 24);
    }
    *reinterpret_cast<v4i*>(wqt + (v0 + vr) * ldx + j0 + jc) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
  }
}

// bf16 operands (the eval head, tiny/train.py:741 under bf16 autocast): no quantisation, only the layout.
// dst [rows_p][cols_p] bf16 = src [rows][cols] rounded to bf16 (RNE, as autocast's cast), zero outside; 8 outputs per thread.
template <typename T>
__global__ __launch_bounds__(256) void prep_x_bf16_kernel(const T* __restrict__ src, int64_t ld, int64_t rows, int64_t cols,
                                                         uint16_t* __restrict__ dst, int64_t rows_p, int64_t cols_p, int64_t dst_ld) {
  const int64_t chunks_per_row = cols_p / 8;
  const int64_t total = rows_p * chunks_per_row;
  for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < total; q += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = q / chunks_per_row, c0 = (q - r * chunks_per_row) * 8;
    uint32_t out[4] = {0, 0, 0, 0};
    if (r < rows) {
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        const uint32_t h = (c0 + m < cols) ? float_to_bf16_bits(Elem<T>::load(src + r * ld + c0 + m)) : 0u;
        out[m >> 1] |= h << (16 * (m & 1));
      }
    }
    *reinterpret_cast<v4i*>(dst + r * dst_ld + c0) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
  }
}

// W (d, V) -> W^T [Vp][dp2 / 2] in bf16 (row stride ldw elements); 64 x 64 tiles through LDS.
template <typename T>
__global__ __launch_bounds__(256) void prep_w_bf16_kernel(const T* __restrict__ w, int64_t ld, int64_t d, int64_t V,
                                                         uint16_t* __restrict__ wt, int64_t ldw) {
  __shared__ uint16_t tile[64][66];
  const int t = threadIdx.x;
  const int64_t j0 = (int64_t)blockIdx.y * 64, v0 = (int64_t)blockIdx.x * 64;
  for (int e = t; e < 64 * 64; e += 256) {
    const int r = e >> 6, c = e & 63;
    tile[r][c] = (j0 + r < d && v0 + c < V) ? float_to_bf16_bits(Elem<T>::load(w + (j0 + r) * ld + v0 + c)) : (uint16_t)0;
  }
  __syncthreads();
  for (int e = t; e < 64 * 64; e += 256) {
    const int vr = e >> 6, jc = e & 63;
    wt[(v0 + vr) * ldw + j0 + jc] = tile[jc][vr];
  }
}

// flat cast, for the standalone sce_quantize_e4m3 entry point
template <typename T>
__global__ __launch_bounds__(256) void quantize_flat_kernel(const T* __restrict__ src, uint8_t* __restrict__ dst,
                                                           size_t n, float inv_scale, const float* __restrict__ scale_dev) {
  const Scaler scale = make_scaler<T>(inv_scale, scale_dev);
  for (size_t q = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; q < n; q += (size_t)gridDim.x * blockDim.x * 4) {
    float v[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) v[m] = (q + m < n) ? scale.apply<T>(Elem<T>::load(src + q + m)) : 0.f;
    const uint32_t w = cvt4_e4m3(v[0], v[1], v[2], v[3]);
    if (q + 4 <= n && (((uintptr_t)(dst + q)) & 3) == 0) {
      *reinterpret_cast<uint32_t*>(dst + q) = w;
    } else {
      for (int m = 0; m < 4 && q + m < n; ++m) dst[q + m] = (uint8_t)(w >> (8 * m));
    }
  }
}

// max |src| over n elements, as the bits of a non-negative float (they order like unsigned integers, NaN above
// everything); *bits starts at 0 (amax_begin_kernel) and ends as max / 448 (amax_end_kernel).
__global__ void amax_begin_kernel(uint32_t* bits) { *bits = 0u; }
template <typename T>
__global__ __launch_bounds__(256) void amax_kernel(const T* __restrict__ src, size_t n, uint32_t* __restrict__ bits) {
  __shared__ uint32_t smax[256];
  uint32_t m = 0u;
  for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < n; q += (size_t)gridDim.x * blockDim.x) {
    const uint32_t b = __float_as_uint(Elem<T>::load(src + q)) & 0x7fffffffu;
    m = b > m ? b : m;
  }
  smax[threadIdx.x] = m;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (threadIdx.x < w) smax[threadIdx.x] = smax[threadIdx.x] > smax[threadIdx.x + w] ? smax[threadIdx.x] : smax[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) atomicMax(bits, smax[0]);
}
__global__ void amax_end_kernel(uint32_t* bits) { *reinterpret_cast<float*>(bits) = __uint_as_float(*bits) / 448.0f; }

// dst (cols, rows) = src (rows, cols)^T, bytes.
__global__ __launch_bounds__(256) void transpose_bytes_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                             int64_t rows, int64_t cols) {
  __shared__ uint8_t tile[64][68];
  const int t = threadIdx.x;
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  for (int e = t; e < 64 * 64; e += 256) {
    const int r = e >> 6, c = e & 63;
    tile[r][c] = (r0 + r < rows && c0 + c < cols) ? src[(r0 + r) * cols + c0 + c] : 0;
  }
  __syncthreads();
  for (int e = t; e < 64 * 64; e += 256) {
    const int c = e >> 6, r = e & 63;
    if (r0 + r < rows && c0 + c < cols) dst[(c0 + c) * rows + r0 + r] = tile[r][c];
  }
}

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
// its own, D_iv 2^{lam_i} is what is stored, with lam_i an integer estimated before the forward pass from a sample of
// the row's logits (fwd_sample_kernel) and undone exactly in rho_i.  The block exponent is taken after the boost, so
// a poor estimate costs precision, never range.
//
// Layout: G^T, tile by tile ([v tile][K block of 128 rows i][256 v][128 i] bytes): the B operand of dW as it lies,
// and of dX through the transposing LDS read.  Exponents: one dword per (128 v, 128 i), byte c for rows [32 c, 32 c + 32),
// as gexp[v / 128][i / 128].
//
// One wave turns its 128 (v) x 128 (i) quadrant of a finished logit tile into its quadrant of the staging tile TT
// ([256 v][STG_PITCH], rows i contiguous) in LDS and returns the dword of exponents of its four 32-row blocks.  The
// transposition happens in registers: the four lanes of a quad hold four consecutive rows of the same four
// columns, and two quad-permute + byte-permute steps turn that 4 x 4 byte block around.
// STATS: the forward pass's row statistics as well (sum of e^{z - cap}, largest raw logit and its column), kept in
// `stat` (LDS, 12 floats per lane: [sum, max, argmax][4 row blocks], NTHREADS apart).
constexpr int STG_PITCH = 272;                               // 256 + 16: 16-byte aligned, rows shifted by 4 banks
constexpr int STG_BYTES = 256 * STG_PITCH;                   // 69632

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

// lam (LDS, wave-uniform base; per row block LAM_STRIDE floats apart, one float for each of LAM_LANES lanes): the row's
// exponent boost (see fwd_sample_kernel).
// want_argmax (uniform, STATS only): see the lookup of the maximum's column below.
template <bool EDGE, bool STATS, int LAM_STRIDE = NTHREADS, int LAM_LANES = 64>
__device__ __forceinline__ uint32_t form_dlogits(const v16f (&acc)[4][4], float k1, float c2, int vlim, int vabs0,
                                                 uint8_t* TT, int wa, int wb, float* stat, const float* lam, bool want_argmax = true) {
  const int lane = lane_id();
  const int vloc0 = wa * 128 + 4 * (lane >> 5);       // column (within the tile) of accumulator register 0 of block a = 0
  const int k = lane & 3;
  const uint32_t sel1 = (k & 1) ? 0x03070105u : 0x06020400u;
  const uint32_t sel2 = (k & 2) ? 0x03020706u : 0x05040100u;
  uint32_t expword = 0;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int iloc = wb * 128 + b * 32 + (lane & 31);        // row within the tile
    // the block's largest logit fixes its exponent: D * 2^s <= 2^(lg + s) <= 446 with lg = log2 e^{zmax - cap}
    float tmax = -INFINITY;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float x = acc[a][b][r];
        if (EDGE && vloc0 + a * 32 + 8 * (r >> 2) + (r & 3) >= vlim) x = -INFINITY;
        tmax = fmaxf(tmax, x);
      }
    const float lamb = lam[b * LAM_STRIDE + (lane_id() & (LAM_LANES - 1))];      // (index taken anew: see lane_id)
    const float lg = wave_max_dpp(fmaf(c2, fast_rcp(1.0f + fast_exp2(tmax * k1)), lamb));      // over the block: log2 of the largest boosted e^{z - cap}
    const float sb = floorf(8.8f - lg);                       // between -120 and 8 + 2 cap log2(e) <= 124 (cap <= 40, boost <= 120)
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
#pragma unroll
        for (int m = g0; m < g0 + NB; ++m) rr[m] = fast_rcp(rr[m] + 1.0f);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = g0; m < g0 + NB; ++m) gg[m] = fast_exp2(fmaf(c2, rr[m], cs));
        __builtin_amdgcn_sched_barrier(0);
        if (EDGE) {
#pragma unroll
          for (int m = g0; m < g0 + NB; ++m) gg[m] = (vloc0 + a * 32 + 8 * (m >> 2) + (m & 3) >= vlim) ? 0.f : gg[m];
        }
        if (STATS) {
#pragma unroll
          for (int m = g0; m < g0 + NB; ++m) ssum += gg[m];
        }
#pragma unroll
        for (int m = g0; m < g0 + NB; ++m) gg[m] *= rr[m] - rr[m] * rr[m];
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int vloc = vloc0 + a * 32 + 8 * q;
        const uint32_t w = cvt4_e4m3(gg[4 * q], gg[4 * q + 1], gg[4 * q + 2], gg[4 * q + 3]);
        // 4 x 4 byte transpose inside the quad: lane k ends up with column vloc + k, rows (iloc & ~3) .. +3
        const uint32_t p1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0xB1, 0xF, 0xF, true);     // lane ^ 1
        const uint32_t x = __builtin_amdgcn_perm(p1, w, sel1);
        const uint32_t p2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, true);     // lane ^ 2
        const uint32_t yv = __builtin_amdgcn_perm(p2, x, sel2);
        *reinterpret_cast<uint32_t*>(TT + (vloc + k) * STG_PITCH + (iloc & ~3)) = yv;
      }
    }
    if (STATS) {
      stat[(0 + b) * NTHREADS] += ssum * fast_exp2(-cs);
      const float amax = stat[(4 + b) * NTHREADS];
      // The column of the maximum is looked up only when a tile reaches a lane's running maximum (on a tie the lower
      // column wins: the running one may be a target of this very tile, which take_target_logits has put there) -- which
      // some lane of the 64 does in nearly every tile of a walk of a few dozen: a caller that does not ask for the argmax
      // is spared it.  (A flag at run time, not a template parameter: without the lookup in the code the register
      // allocation of the rest changes, and accumulators end up in scratch memory.)
      if (want_argmax && __builtin_amdgcn_ballot_w64(tmax >= amax) != 0) {
        if (tmax >= amax) {
          int targ = 0x7fffffff;
#pragma unroll
          for (int a = 3; a >= 0; --a) {
#pragma unroll
            for (int r = 15; r >= 0; --r) {
              const int vo = a * 32 + 8 * (r >> 2) + (r & 3);
              if (acc[a][b][r] == tmax && (!EDGE || vloc0 + vo < vlim)) targ = vo;   // descending scan: lowest column wins
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

// The wave's quadrant of the staging tile (128 columns v x 128 rows i) is one contiguous 16 KB run of G^T: out in
// 16-byte stores.  A wave reads only what it wrote itself, so no barrier is needed between forming and storing.
__device__ __forceinline__ void store_dlogits_quadrant(const uint8_t* TT, uint8_t* gcol, int wa, int wb) {
  const int lane = lane_id();
  const uint8_t* tq = TT + wa * 128 * STG_PITCH + wb * 128;
#pragma unroll
  for (int n = 0; n < 16; ++n) {
    const int cidx = lane + 64 * n, row = cidx >> 3, col = (cidx & 7) * 16;
    *reinterpret_cast<v4i*>(gcol + row * BK + col) = *reinterpret_cast<const v4i*>(tq + row * STG_PITCH + col);
  }
}

// ------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------
struct FwdParams {
  const uint8_t* xq;       // [Np][dp]
  const uint8_t* wqt;      // [Vp][dp]
  float4* partials;        // [S][Np]: sum exp(z - cap), max u, argmax u (bits), unused
  const int64_t* targets;  // (N,)
  float* s_uy;             // [n_predict][Np]: raw logit u at the target of (offset, row), written by the workgroup that meets it
  uint8_t* ghat_t;         // EMIT: G^T, all Np rows (K blocks per v tile: kbw)
  uint32_t* gexp;          // EMIT: its block exponents [Vp / 128][kbw]
  const float* lam;        // EMIT: exponent boost of every row
  int64_t ignore_index;
  int64_t dp, ldx;         // K extent and row stride of xq / wqt
  int64_t kbw;
  int N, V, Np, RT, CT, S, n_predict;      // V: columns that take part; CT: column tiles walked (EMIT: all of Vp / 256)
  float sc;                // x_s * w_s
  float k1;                // x_s * w_s * 2 log2(e) / cap : exp2(acc * k1) = e^{2u/cap}
  float ic2;               // 1 / c2, c2 = -2 cap log2(e): e^{z - cap} = exp2(c2 / (1 + e^{2u/cap}))
  float c2;
  const DevConsts* dc;     // non-NULL: sc and k1 come from here (a scale lives on the device)
  int want_argmax;         // the caller asks for the rows' argmax: the column of the running maximum is tracked
};

// Per 256 x 256 tile and per row a lane owns: add up e^{z - cap} over its 64 columns and keep the
// largest raw accumulator.  z is bounded by +-cap, so no running maximum is needed for the sum:
//   t = tanh(u/cap) = 1 - 2/(E + 1), E = e^{2u/cap};   e^{z - cap} = exp2(c2 / (E + 1)).
// The column of the maximum is looked up only on the (rare, after the first tiles) occasion that
// a tile raises a row's running maximum.
// ROUND: the logits are rounded to bf16 first (bf16 operands: the GEMM of the eager head returns bf16).
template <bool EDGE, bool ROUND = false>
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
        float x = ROUND ? round_to_bf16(acc[a][b][r]) : acc[a][b][r];
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
            if ((ROUND ? round_to_bf16(acc[a][b][r]) : acc[a][b][r]) == tmax && (!EDGE || vo < p.V - vbase)) targ = vo;   // descending scan: lowest column wins
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
// and lse come from the same numbers: the fp8 matrix instruction sums with less than fp32 care (about 2e-5 low on a
// sum of like-signed terms), and a z_y from a separate fp32 dot product would leave that bias in z_y - lse, i.e. in
// 1 - p_y, where rows the model is sure of cannot afford it.  tgt (LDS): [4 offsets][TGT_STRIDE rows] target column or
// -1, already at the wave's first row.  A lane looks at its four rows; the 64-way select runs only when some lane of
// the wave has a hit (a few per cent of the tiles).
// STORE: the logit goes to s_uy_tile[offset][row] (global).
// KNOCK: the accumulator of the target is then set to -inf, for the dlogits epilogue that follows: the target takes
//        no part in the stored dlogits (its column is handled in fp32, see bwd_prep_kernel) and must not set the
//        exponent of its block either -- a row the model is sure of would push its own other columns, and its
//        neighbours', out of the 8 bits.
// STATS: with KNOCK, the row statistics (stat, as in form_dlogits) take the target's share here: e^{z_y - cap} into the
//        sum, and the running maximum / argmax.
template <bool STORE, bool KNOCK, bool STATS, int TGT_STRIDE, bool ROUND = false>
__device__ __forceinline__ void take_target_logits(v16f (&acc)[4][4], const int* tgt, int n_predict, int col0, int rowbase,
                                                   float sc, float* s_uy_tile, int Np, float* stat, float k1, float ic2) {
  const int lane = lane_id(), half = lane >> 5;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
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
              stat[(0 + b) * NTHREADS] += fast_exp2(fast_rcp(fmaf(fast_exp2(x * k1), ic2, ic2))) - fast_exp2(fast_rcp(ic2));
              const float amax = stat[(4 + b) * NTHREADS];
              if (x > amax || (x == amax && y < __float_as_int(stat[(8 + b) * NTHREADS]))) {
                stat[(4 + b) * NTHREADS] = x;
                stat[(8 + b) * NTHREADS] = __int_as_float(y);
              }
            }
          }
          xk[k] = x;
          // (the lane index is taken anew: an address kept from outside the branch stays live across the main loop and is spilled)
          if (STORE) s_uy_tile[(int64_t)k * Np + rowbase + b * 32 + (lane_id() & 31)] = ROUND ? round_to_bf16(x) * sc : x * sc;
        }
      }
    }
  }
}

// The exponent boost of every row, from one tile of its logits (256 columns from the middle of the vocabulary):
// lam_i = floor(-log2 m_i), m_i the smallest of the means of e^{z - cap} over 16 groups of 16 columns -- the smallest,
// so that a few peaks inside the sample (a target, say) do not pass for the level of the row.  One workgroup per row tile.
__global__ __launch_bounds__(256) void fwd_sample_kernel(FwdParams p_in, int ct, float* __restrict__ lam_out) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  FwdParams p = p_in;
  if (p.dc) { p.sc = p.dc->sc; p.k1 = p.dc->k1; }
  const int rt = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wa = wave >> 1, wb = wave & 1;
  v16f acc[4][4];
  mfma_mainloop(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, p.xq + (int64_t)rt * 256 * p.ldx, p.ldx, (int)(p.dp / BK), smem, acc, 0, 0, wave);
  const int lane = lane_id();
  const int vlim = p.V - ct * 256, vloc0 = wa * 128 + 4 * (lane >> 5);
  float gmin[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    gmin[b] = INFINITY;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      float sum = 0.f, cnt = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pt = fast_exp2(fast_rcp(fmaf(fast_exp2(acc[a][b][r] * p.k1), p.ic2, p.ic2)));
        const bool live = vloc0 + a * 32 + 8 * (r >> 2) + (r & 3) < vlim;
        sum += live ? pt : 0.f;
        cnt += live ? 1.f : 0.f;
      }
      if (cnt > 0.f) gmin[b] = fminf(gmin[b], sum / cnt);
    }
    gmin[b] = fminf(gmin[b], __shfl_xor(gmin[b], 32));
  }
  float* red = reinterpret_cast<float*>(smem);          // free: the main loop has ended in every wave
  if (wa == 1 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 4; ++b) red[wb * 128 + b * 32 + lane] = gmin[b];
  }
  __syncthreads();
  if (wa == 0 && lane < 32) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float m = fminf(gmin[b], red[wb * 128 + b * 32 + lane]);
      float l = floorf(-log2f(m));
      l = l > 0.f ? (l < 120.f ? l : 120.f) : 0.f;           // also: NaN -> 0
      lam_out[rt * 256 + wb * 128 + b * 32 + lane] = l;
    }
  }
}

// LDS of the forward kernel: the two K slots; with EMIT the staging tile of the dlogits in the second slot (reaching
// 4 KB beyond it); the row statistics of the workgroup's walk (12 values per lane, and the boosts of its rows: kept in registers they are spilled
// around the main loop, and the reload -- a vector memory load -- makes the epilogue wait for the tile loads that were
// just put in flight for the next tile); the targets of the workgroup's 256 rows.
constexpr int FWD_STAGE_OFF = SLOT_BYTES;
constexpr int FWD_STAT_OFF = SMEM_MAX - 4096 - 16 * 4 * NTHREADS;      // 12 statistics and the boosts of the lane's 4 rows
constexpr int FWD_TGT_OFF = SMEM_MAX - 4096;
constexpr int SMEM_FWD = SMEM_MAX;
static_assert(FWD_STAGE_OFF + STG_BYTES <= FWD_STAT_OFF, "staging tile and row statistics overlap");

// EMIT: the epilogue also leaves the block-scaled dlogits of the tile in G^T (see form_dlogits), for a backward pass
// that does not compute the logits again.
// BF16 (without EMIT): bf16 operands, logits rounded to bf16 as the eager head's GEMM returns them (forward only).
template <bool EMIT, bool BF16 = false>
__global__ __launch_bounds__(256) void fwd_kernel(FwdParams p_in) {
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
    }
  }
  __syncthreads();
  v16f acc[4][4];
  const uint8_t* Bg = p.xq + (int64_t)rt * 256 * p.ldx;
  const int KT = (int)(p.dp / BK);
  // of the workgroups that start together on this XCD, those with the same split share the W tiles, those with the same rt the X rows
  const int rot_a = 2 * (rt & 3), rot_b = s & 7;
  // the first K blocks of the next tile travel while the epilogue of this one runs (it does not touch the K slots;
  // with EMIT it uses the second one, so only the first block travels and the rest follows after the epilogue)
  if (ct0 < ct1) mfma_prefetch(p.wqt + (int64_t)ct0 * 256 * p.ldx, p.ldx, Bg, p.ldx, smem, rot_a, rot_b, wave);
  for (int ct = ct0; ct < ct1; ++ct) {
    mfma_mainloop<true, NoHook, BK, false, 0, BF16>(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, Bg, p.ldx, KT, smem, acc, rot_a, rot_b, wave,
                                                    NoHook(), 0, 0, nullptr, EMIT && ct > ct0);
    const uint8_t* Anext = p.wqt + (int64_t)(ct + 1) * 256 * p.ldx;
    if (ct + 1 < ct1) mfma_prefetch<EMIT ? 1 : 3>(Anext, p.ldx, Bg, p.ldx, smem, rot_a, rot_b, wave);
    float* stat = reinterpret_cast<float*>(smem + FWD_STAT_OFF) + wave * 64 + lane_id();
    const int vbase = ct * 256 + wa * 128 + 4 * (lane_id() >> 5);
    const int* tgt = reinterpret_cast<const int*>(smem + FWD_TGT_OFF) + wb * 128;
    if (EMIT) {
      take_target_logits<true, true, true, 256>(acc, tgt, p.n_predict, ct * 256 + wa * 128, rt * 256 + wb * 128, p.sc, p.s_uy, p.Np, stat, p.k1, p.ic2);
      const int vlim = p.V - ct * 256;
      uint8_t* TT = smem + FWD_STAGE_OFF;
      uint32_t ew;
      const float* lam = reinterpret_cast<const float*>(smem + FWD_STAT_OFF) + 12 * NTHREADS + wave * 64;
      if (vlim < 256) ew = form_dlogits<true, true>(acc, p.k1, p.c2, vlim, vbase, TT, wa, wb, stat, lam, p.want_argmax != 0);
      else ew = form_dlogits<false, true>(acc, p.k1, p.c2, vlim, vbase, TT, wa, wb, stat, lam, p.want_argmax != 0);
      store_dlogits_quadrant(TT, p.ghat_t + ((int64_t)ct * p.kbw + 2 * rt + wb) * BLOCKED_KSTEP + wa * 128 * BK, wa, wb);
      if (lane_id() == 0) p.gexp[(int64_t)(2 * ct + wa) * p.kbw + 2 * rt + wb] = ew;
    } else {
      float sum[4], amax[4];
      int uarg[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        sum[b] = stat[(0 + b) * NTHREADS]; amax[b] = stat[(4 + b) * NTHREADS]; uarg[b] = __float_as_int(stat[(8 + b) * NTHREADS]);
      }
      if (ct * 256 + 256 > p.V) fwd_epilogue<true, BF16>(acc, p, vbase, sum, amax, uarg);
      else fwd_epilogue<false, BF16>(acc, p, vbase, sum, amax, uarg);
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        stat[(0 + b) * NTHREADS] = sum[b]; stat[(4 + b) * NTHREADS] = amax[b]; stat[(8 + b) * NTHREADS] = __int_as_float(uarg[b]);
      }
    }
    if (!EMIT) take_target_logits<true, false, false, 256, BF16>(acc, tgt, p.n_predict, ct * 256 + wa * 128, rt * 256 + wb * 128, p.sc, p.s_uy, p.Np, nullptr, 0.f, 0.f);
    if (EMIT && ct + 1 < ct1) {
      // every wave has read its part of the staging tile (its stores have their data) before the second K slot fills again
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      mfma_prefetch<2>(Anext, p.ldx, Bg, p.ldx, smem, rot_a, rot_b, wave);
    }
  }
  if (EMIT) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");     // the staging tile gives way to the reduction below
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
                                                      float* __restrict__ blockmax, int32_t* __restrict__ rowinfo) {
  __shared__ float smax[256];
  const int i = blockIdx.x * 256 + threadIdx.x;
  float r = 0.f;
  float h[4] = {0.f, 0.f, 0.f, 0.f};
  if (rowinfo && i < Np) {          // what the recompute kernel wants to know of a row: its boost and its target columns
    rowinfo[i] = __float_as_int(i < N ? lam[i] : 0.f);
    for (int k = 0; k < 4; ++k)
      rowinfo[(int64_t)(1 + k) * Np + i] = (k < n_predict && i < N && target_valid(targets, ignore_index, i + k, N, V)) ? (int)targets[i + k] : -1;
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
      r = ldexpf(g * sw * expf(cap - lse), -(int)lam[i]);      // the stored dlogits carry the row's boost 2^lam
    }
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

// Xt (blocked, dq rows, K = Np) = e4m3( X_q[i][j] * rho_i / xi ), transposed through LDS in 64 x 64 tiles.
__global__ __launch_bounds__(256) void bwd_xt_kernel(const uint8_t* __restrict__ xq, int64_t dp, int64_t ldx, int64_t kbn,
                                                    const float* __restrict__ rho, const float* __restrict__ xi,
                                                    uint8_t* __restrict__ xt) {
  __shared__ uint8_t tile[64][68];
  const int t = threadIdx.x;
  const int64_t i0 = (int64_t)blockIdx.x * 64, j0 = (int64_t)blockIdx.y * 64;
  if (j0 < dp) {
    const int r = t >> 2, c = (t & 3) * 16;
    const v4i raw = *reinterpret_cast<const v4i*>(xq + (i0 + r) * ldx + j0 + c);
    const float f = rho[i0 + r] / xi[0];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const uint32_t w = (uint32_t)raw[m];
      const uint32_t o = cvt4_e4m3(e4m3_to_float<0>(w) * f, e4m3_to_float<1>(w) * f, e4m3_to_float<2>(w) * f,
                                   e4m3_to_float<3>(w) * f);
      *reinterpret_cast<uint32_t*>(&tile[r][c + 4 * m]) = o;
    }
  } else {
    for (int e = t; e < 64 * 17; e += 256) reinterpret_cast<uint32_t*>(&tile[0][0])[e] = 0;
  }
  __syncthreads();
  const int jr = t >> 2, ic = (t & 3) * 16;
  uint32_t out[4];
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    out[m] = (uint32_t)tile[ic + 4 * m][jr] | ((uint32_t)tile[ic + 4 * m + 1][jr] << 8) |
             ((uint32_t)tile[ic + 4 * m + 2][jr] << 16) | ((uint32_t)tile[ic + 4 * m + 3][jr] << 24);
  }
  *reinterpret_cast<v4i*>(xt + blocked_offset(j0 + jr, i0 + ic, kbn)) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
}

struct RecomputeParams {
  const uint8_t* xq;     // [Np][dp], already offset to the panel's first row
  const uint8_t* wqt;    // [Vp][dp]
  uint8_t* ghat_t;       // Vp rows, K = 128 * kbw, blocked
  uint32_t* gexp;        // [Vp / 128][kbw]
  const int32_t* rowinfo;      // [ROWINFO_PLANES][Np], offset to the panel's first row: boosts and targets (bwd_prep_kernel)
  int64_t Np;
  int n_predict;
  int64_t dp, ldx;             // K extent and row stride of xq / wqt
  int64_t kbw, kb0;            // ghat_t (blocked): K blocks per tile, K block of this panel's first row
  int RT, CT, V;
  float k1, c2;          // as in FwdParams
  const DevConsts* dc;   // non-NULL: k1 comes from here
};

// Recompute a 256 x 256 logit tile and leave its block-scaled dlogits in G^T.  The tile is assembled in LDS (free
// once the main loop is done) and leaves the chip as 64 KB of consecutive 16-byte stores.
constexpr int ROWINFO_PLANES = 5;                      // per row: exponent boost (a float), then the target column of each of 4 offsets (or -1)
constexpr int SMEM_RECOMPUTE = SMEM_BYTES + 4 * ROWINFO_PLANES * 512;      // two K slots (the staging tile reuses them) + the row data of 128 rows per wave
static_assert(STG_BYTES <= SMEM_BYTES, "the staging tile must fit the K slots");

__global__ __launch_bounds__(256) void bwd_recompute_kernel(RecomputeParams p_in) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  RecomputeParams p = p_in;
  if (p.dc) p.k1 = p.dc->k1;
  int rt, ct;
  if (!map_tile(blockIdx.x, p.RT, p.CT, rt, ct)) return;
  // The tile order goes through the columns in groups of 8, and it does so from the last group to the first:
  // the dX kernel that follows starts its K loop at column 0, with the part of G that was written last and is
  // still in the memory-side cache.
  ct = p.CT - 1 - ct;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wa = wave >> 1, wb = wave & 1;
  // The boosts and targets of the wave's 128 rows go straight to LDS, behind the two slots: requested before the K
  // loop (whose waits for its own, younger loads cover them), read after it, no register held in between.
  {
    const uint32_t dst = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)(smem + SMEM_BYTES)) + wave * (ROWINFO_PLANES * 512);
    const int voff = lane_id() * 4;
#pragma unroll
    for (int q = 0; q < ROWINFO_PLANES; ++q) {
      const int32_t* src = p.rowinfo + (int64_t)q * p.Np + rt * 256 + wb * 128;
      // the instruction's offset moves the memory address and the LDS address alike: the second half of the rows
      asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3\n\t"
                   "global_load_lds_dword %2, %3 offset:256"
                   ::"s"(dst), "n"(q * 512), "v"(voff), "s"(src) : "memory", "scc");
    }
  }
  v16f acc[4][4];
  mfma_mainloop(p.wqt + (int64_t)ct * 256 * p.ldx, p.ldx, p.xq + (int64_t)rt * 256 * p.ldx, p.ldx, (int)(p.dp / BK), smem, acc, 2 * (rt & 3), ct & 7, wave);
  const int vlim = p.V - ct * 256;           // columns >= vlim of this tile do not exist
  const float* lam = reinterpret_cast<const float*>(smem + SMEM_BYTES) + wave * (ROWINFO_PLANES * 128);     // row block b: 32 floats on
  const int* tgt = reinterpret_cast<const int*>(smem + SMEM_BYTES) + wave * (ROWINFO_PLANES * 128) + 128;
  take_target_logits<false, true, false, 128>(acc, tgt, p.n_predict, ct * 256 + wa * 128, 0, 0.f, nullptr, 0, nullptr, 0.f, 0.f);
  uint32_t ew;
  if (vlim < 256) ew = form_dlogits<true, false, 32, 32>(acc, p.k1, p.c2, vlim, 0, smem, wa, wb, nullptr, lam);
  else ew = form_dlogits<false, false, 32, 32>(acc, p.k1, p.c2, vlim, 0, smem, wa, wb, nullptr, lam);
  store_dlogits_quadrant(smem, p.ghat_t + ((int64_t)ct * p.kbw + p.kb0 + 2 * rt + wb) * BLOCKED_KSTEP + wa * 128 * BK, wa, wb);
  if (lane_id() == 0) p.gexp[(int64_t)(2 * ct + wa) * p.kbw + p.kb0 + 2 * rt + wb] = ew;
}

struct DxParams {
  const uint8_t* wq;      // dq rows, K = Vp, tile by tile: A side (rows j)
  const uint8_t* ghat_t;  // G^T, blocked; already at the K block of the panel's first row    B side (rows i of the panel)
  const uint32_t* gexp;   // its block exponents [Vp / 128][kbw], likewise at the panel's first row
  const uint8_t* wqt;     // [Vp][dp]   for the one-hot gather
  const float* rho;       // offset to the panel
  const float* hcoef;     // [n_predict][Np], offset to the panel
  const int64_t* targets; // offset to the panel
  void* dx;               // offset to the panel's first row
  float* part;            // [ksplit][RT * 256][dq] fp32 partial sums (ksplit > 1 only)
  int64_t dx_ld, Vp, ldx, Np, dq;        // Vp: K extent; ldx: row stride of wqt
  int64_t kbw;                           // K blocks (of 128 rows i) per v tile of ghat_t
  int RT, CT, rows, d, V;  // rows: valid rows in this panel
  int n_predict, rows_left; // rows_left: N - (first row of the panel), bounds the target look-ahead
  int ksplit;              // the K loop (V) is cut into this many parts, one workgroup each
  float w_s;
  const DevConsts* dc;     // non-NULL: w_s comes from here
};

// Row scale and one-hot term of four consecutive dX columns j..j+3 of panel row il:
//   dX = rho_i w_s (G W_q^T) - sum_k h_ik w_s W_q^T[y_{i+k}, :]
// LDS a wave uses to stage its quadrant of a dX tile on the way out: 128 rows of 64 fp32 (or bf16) plus 16 bytes
constexpr int DX_STAGE_BYTES = 128 * (64 * 4 + 16);
constexpr int SMEM_DX = 4 * DX_STAGE_BYTES > SMEM_BYTES ? 4 * DX_STAGE_BYTES : SMEM_BYTES;
// ... or the two K slots and, behind them, the block exponents of the K loop (one dword per K block and half of the rows)
constexpr int MAX_SCALE_KBLOCKS = (SMEM_MAX - SMEM_BYTES) / 8;      // K blocks of one scaled main loop: 4096
static inline int smem_scaled(int kblocks, int at_least) { const int n = SMEM_BYTES + 8 * kblocks; return n > at_least ? n : at_least; }

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
  // B = G^T: K (v) is the slow index there.  The 128 v rows of a K block are half a v tile; the 256 panel rows of this
  // tile are the two 128-byte pieces of i blocks 2 rt and 2 rt + 1 (BLOCKED_KSTEP apart).
  const int64_t bpair = p.kbw * BLOCKED_KSTEP;                     // from one v tile (two K blocks) to the next
  mfma_mainloop<false, NoHook, BLOCKED_KSTEP, true, 1>(p.wq + ((int64_t)ct * (p.Vp / BK) + k0 / BK) * BLOCKED_KSTEP, BK,
                                                       p.ghat_t + 2 * (int64_t)rt * BLOCKED_KSTEP + (k0 / (2 * BK)) * bpair, BLOCKED_KSTEP, KD, smem, acc,
                                                       2 * (rt & 3), ct & 7, __builtin_amdgcn_readfirstlane(wave), NoHook(), 128 * BK, bpair,
                                                       lsc + __builtin_amdgcn_readfirstlane(wb) * KD);
  const int jbase = ct * 256 + wa * 128 + 4 * (lane >> 5);
  T* dx = reinterpret_cast<T*>(p.dx);
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
  const uint8_t* ghat_t;  // Vp rows, blocked, already at the first K block of this launch          B side (rows v)
  const uint32_t* gexp;   // its block exponents [Vp / 128][kbw], likewise
  float* dwacc;           // [dq][Vp] fp32
  int64_t kbn, kbw, kb0, Vp;   // K blocks per tile of xt and of ghat_t; first K block of xt in this launch; row length of dwacc
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
  mfma_mainloop<false, NoHook, BLOCKED_KSTEP, false, 2>(p.xt + ((int64_t)rt * p.kbn + p.kb0) * BLOCKED_KSTEP, BK, p.ghat_t + (int64_t)ct * p.kbw * BLOCKED_KSTEP, BK, p.KT,
                                                        smem, acc, ct & 7, 2 * (rt & 3), __builtin_amdgcn_readfirstlane(wave), NoHook(), 0, 0,
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

// sort keys: one entry per (offset k, row i): key = target y_{i+k} (V if the pair takes no part; targets at or
// beyond the vocabulary limit Vl take no part),
// value = entry id k * Np + i
// The tiles of the last, partly filled round of dW (tile0 .. tile0 + ntail - 1 of the round-robin order), shared out
// along K: a tile's K loop is kp pairs of K blocks long, all of them together W = ntail * kp pairs, and workgroup g takes
// pairs [g share, (g + 1) share) of that line -- the end of one tile and the beginning of the next, when its range
// straddles them.  Piece (g, t) of tile t goes to buf[g + t] as plain stores (g + t grows by one from each piece to the
// next along the line, so no two pieces meet); bwd_dw_final_kernel adds up a tile's pieces in the order of g.
// a pointer that is the same in every lane, moved to scalar registers
__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* q) {
  const uint64_t u = (uint64_t)(uintptr_t)q;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)u), hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(u >> 32));
  return (const uint8_t*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
struct DwTail {
  float* buf;
  int tile0, ntail, kp, share;      // tile0 < 0: no tail (every tile is in the fp32 partial)
};
__global__ __launch_bounds__(256) void bwd_dw_tail_kernel(DwParams p, DwTail tl) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int g = blockIdx.x;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wa = wave >> 1, wb = wave & 1;
  int pos = g * tl.share;
  const int end = min(tl.ntail * tl.kp, pos + tl.share);
  uint32_t* lsc = reinterpret_cast<uint32_t*>(smem + SMEM_BYTES);
  while (pos < end) {
    // (everything here is uniform, but the divisions leave their results in vector registers: the main loop wants
    // its addresses in scalar ones)
    const int tt = __builtin_amdgcn_readfirstlane(pos / tl.kp);
    const int k0 = pos - tt * tl.kp, k1 = min(tl.kp, k0 + (end - pos)), KD = 2 * (k1 - k0);
    int rt, ct;
    tile_from_index(tl.tile0 + tt, p.RT, p.CT, rt, ct);
    rt = __builtin_amdgcn_readfirstlane(rt); ct = __builtin_amdgcn_readfirstlane(ct);
    for (int e = t; e < 2 * KD; e += NTHREADS) {
      const int w = e >= KD, kb = e - w * KD;
      lsc[e] = p.gexp[(int64_t)(2 * ct + w) * p.kbw + 2 * k0 + kb];
    }
    __syncthreads();
    v16f acc[4][4];
    mfma_mainloop<false, NoHook, BLOCKED_KSTEP, false, 2>(uniform_ptr(p.xt + ((int64_t)rt * p.kbn + p.kb0 + 2 * k0) * BLOCKED_KSTEP), BK,
                                                          uniform_ptr(p.ghat_t + ((int64_t)ct * p.kbw + 2 * k0) * BLOCKED_KSTEP), BK,
                                                          __builtin_amdgcn_readfirstlane(KD), smem, acc, ct & 7, 2 * (rt & 3),
                                                          __builtin_amdgcn_readfirstlane(wave), NoHook(), 0, 0,
                                                          lsc + __builtin_amdgcn_readfirstlane(wb) * KD);
    float* dst0 = tl.buf + (size_t)(g + tt) * 65536 + (wa * 128 + 4 * (lane >> 5)) * 256 + wb * 128 + (lane & 31);
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) dst0[(a * 32 + 8 * (r >> 2) + (r & 3)) * 256 + b * 32] = acc[a][b][r];
    pos += k1 - k0;
  }
}

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

}  // namespace sce

// ==========================================================================================
// host side: C ABI
// ==========================================================================================
namespace sce {
int sort_pairs(void* tmp, size_t* tmp_bytes, const int32_t* kin, int32_t* kout, const int32_t* vin, int32_t* vout,
               size_t n, int end_bit, hipStream_t stream);   // sce_sort.hip
}

using namespace sce;

static thread_local char g_err[512] = "";

static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define HIP_TRY(expr)                                                                              \
  do {                                                                                             \
    hipError_t e_ = (expr);                                                                        \
    if (e_ != hipSuccess) return fail(SCE_EHIP, "%s failed: %s", #expr, hipGetErrorString(e_));    \
  } while (0)

struct DeviceGuard {
  int prev = -1;
  bool ok = true;
  explicit DeviceGuard(int dev) {
    if (hipGetDevice(&prev) != hipSuccess) { ok = false; return; }
    if (prev != dev && hipSetDevice(dev) != hipSuccess) ok = false;
  }
  ~DeviceGuard() { if (prev >= 0) (void)hipSetDevice(prev); }
};

// Scratch of sce_forward_noalloc: the V-split partial records of the forward kernel (what sce_forward takes from the
// caller's workspace).  Every GPU the library runs on holds its own copy until the process ends; in host code the
// array's name is only a handle, the address on a device comes from hipGetSymbolAddress (g_scratch, below).
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

static std::mutex g_mu;
static int g_arch_ok[64];   // 0 unknown, 1 gfx950, -1 other
static void* g_scratch[64]; // device address of `scratch` on each device, filled with g_arch_ok
static int g_cus[64];       // compute units, filled with g_arch_ok
static inline int device_cus_or_default(int dev) { return (dev >= 0 && dev < 64 && g_cus[dev] > 0) ? g_cus[dev] : 256; }

// Optional per-kernel timing with HIP events on the caller's stream (off by default).
struct TimingState {
  bool on = false;
  std::vector<hipEvent_t> pool;                       // unused events
  std::vector<hipEvent_t> begin[SCE_K_COUNT], end[SCE_K_COUNT];
  double ms[SCE_K_COUNT] = {0};
  int64_t launches[SCE_K_COUNT] = {0};
};
static TimingState g_timing;
static std::mutex g_timing_mu;

static hipEvent_t timing_event() {
  if (!g_timing.pool.empty()) { hipEvent_t e = g_timing.pool.back(); g_timing.pool.pop_back(); return e; }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}
struct KernelTimer {   // records an event pair around the launches made while it lives
  int kind; hipStream_t st; bool active;
  KernelTimer(int k, hipStream_t s) : kind(k), st(s), active(false) {
    std::lock_guard<std::mutex> lk(g_timing_mu);
    if (!g_timing.on) return;
    hipEvent_t e = timing_event();
    if (!e) return;
    (void)hipEventRecord(e, st);
    g_timing.begin[kind].push_back(e);
    active = true;
  }
  ~KernelTimer() {
    if (!active) return;
    std::lock_guard<std::mutex> lk(g_timing_mu);
    hipEvent_t e = timing_event();
    if (!e) { g_timing.pool.push_back(g_timing.begin[kind].back()); g_timing.begin[kind].pop_back(); return; }
    (void)hipEventRecord(e, st);
    g_timing.end[kind].push_back(e);
  }
};

// First use of a device: its architecture, and the kernels' LDS limits, set with that device current.  A device
// counts as known only once every step has succeeded, so a failure here is tried again on the next call.
static int check_device(int dev) {
  if (dev < 0 || dev >= 64) return fail(SCE_EINVAL, "device %d out of range", dev);
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_arch_ok[dev] == 0) {
    DeviceGuard guard(dev);
    if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", dev);
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
      g_arch_ok[dev] = -1;
    } else {
      // the MFMA kernels hold two 64 KB K-slots in LDS, and more behind them
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_kernel<false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_pp_kernel<12, false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD_PP));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_pp_kernel<12, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_FWD_PP));
      HIP_TRY(hipFuncSetAttribute((const void*)fwd_sample_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_recompute_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_RECOMPUTE));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<float, false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<bf16_t, false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<float, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dx_kernel<bf16_t, true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dw_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dw_tail_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      HIP_TRY(hipFuncSetAttribute((const void*)bwd_dw_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_MAX));
      void* sp = nullptr;
      HIP_TRY(hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)));       // this device's copy of the array
      g_scratch[dev] = sp;
      g_cus[dev] = prop.multiProcessorCount;
      g_arch_ok[dev] = 1;
    }
  }
  if (g_arch_ok[dev] != 1) return fail(SCE_EARCH, "device %d is not gfx950", dev);
  return SCE_OK;
}

static int check_shape(const sce_shape* s) {
  if (!s) return fail(SCE_EINVAL, "shape is NULL");
  if (s->N <= 0 || s->d <= 0 || s->V <= 0) return fail(SCE_EINVAL, "N, d, V must be positive (got %lld, %lld, %lld)",
                                                       (long long)s->N, (long long)s->d, (long long)s->V);
  if (s->d % 16 != 0) return fail(SCE_EINVAL, "d = %lld must be a multiple of 16", (long long)s->d);
  if (s->N > (1ll << 24) - 256 || s->V > (1ll << 24) - 256 || s->d > (1ll << 24) - 256)
    return fail(SCE_EINVAL, "N, d and V must be below 2^24 (32-bit tile offsets)");
  if (s->V > (int64_t)MAX_SCALE_KBLOCKS * BK)
    return fail(SCE_EINVAL, "V = %lld must be at most %d (the block exponents of a dX tile's K loop wait in LDS)", (long long)s->V, MAX_SCALE_KBLOCKS * BK);
  if (s->d > (1ll << 22) - 256) return fail(SCE_EINVAL, "d = %lld must be below 2^22 (a grid dimension of the layout kernels)", (long long)s->d);
  if (s->n_predict < 1 || s->n_predict > 4) return fail(SCE_EINVAL, "n_predict = %d must be between 1 and 4", s->n_predict);
  return SCE_OK;
}

static size_t sort_tmp_bytes(int64_t N, int64_t V) {
  size_t bytes = 0;
  int bits = 1;
  while ((1ll << bits) <= V) ++bits;
  (void)sce::sort_pairs(nullptr, &bytes, nullptr, nullptr, nullptr, nullptr, (size_t)N, bits, nullptr);
  return bytes;
}

// fp32 partial sums of a K-split dX panel: at most 256 tiles of 256 x 256
constexpr size_t DX_PART_BYTES = (size_t)256 * 256 * 256 * 4;

// The last round of dW tiles, when it is far from full, is shared out along K among DW_TAIL_WGS workgroups
// (bwd_dw_tail_kernel); each leaves its piece of a tile as a 256 x 256 fp32 partial.  A workgroup's range can end inside
// one tile and go on in the next, so there are fewer pieces than workgroups plus tiles.
constexpr int DW_TAIL_WGS = 256;
struct DwTailPlan {
  int full, ntail, kp, share;      // tiles in full rounds, tiles of the last round, pairs of K blocks per tile and per workgroup
  bool use;                        // measured: worth it when the shared-out round is at most half a tile long per workgroup
  size_t bytes;                    // partial tiles: one per (workgroup, tile it touches)
};
static DwTailPlan dw_tail_plan(int64_t dq, int64_t Vp, int64_t krows) {
  DwTailPlan t;
  const int tiles = (int)((dq / 256) * (Vp / 256));
  t.kp = (int)(krows / BK / 2);
  t.full = tiles / DW_TAIL_WGS * DW_TAIL_WGS;
  t.ntail = tiles - t.full;
  t.share = t.ntail > 0 ? (int)(((int64_t)t.ntail * t.kp + DW_TAIL_WGS - 1) / DW_TAIL_WGS) : 0;
  t.use = t.ntail > 0 && t.share >= 1 && t.share * 2 <= t.kp;
  t.bytes = t.use ? (size_t)(DW_TAIL_WGS + t.ntail) * 256 * 256 * 4 : 0;
  return t;
}

// kept: the dlogits come with `saved` (the forward pass emitted them): no panel scratch here
static BwdLayout bwd_layout(const SavedLayout& S, int64_t P, int64_t Pw, int nparts, int K, bool kept = false) {
  BwdLayout B;
  B.P = P; B.Pw = Pw; B.nparts = nparts;
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t r = o; o += (bytes + 255) / 256 * 256; return r; };
  B.off_rho = take((size_t)S.Np * 4);
  B.off_rowinfo = take((size_t)S.Np * 4 * ROWINFO_PLANES);
  B.off_hcoef = take((size_t)S.Np * 4 * K);
  B.off_blockmax = take((size_t)(S.Np / 256) * 4);
  B.off_xi = take(256);
  B.off_xt = take((size_t)S.dq * S.Np);
  B.off_perm = take((size_t)S.N * K * 4 * 2);  // sorted values + unsorted values, one entry per (offset, row)
  B.off_keys = take((size_t)S.N * K * 4 * 2);  // sorted keys + unsorted keys
  B.off_segoff = take((size_t)(S.V + 2) * 4);
  B.off_longlist = take((size_t)(2 * (S.N * K / LONG_SEG + 1) + 2) * 4);   // (column, chunk) pairs: at most one per LONG_SEG entries
  B.off_longbase = take((size_t)S.V * 4);                                  // first slot of each long column
  B.off_longsum = take((size_t)(S.N * K / LONG_SEG + 1) * S.dq * 4);      // chunk sums: a long column has at most one chunk per LONG_SEG of its entries
  B.sorttmp_bytes = sort_tmp_bytes(S.N * K, S.V);
  B.off_sorttmp = take(B.sorttmp_bytes);
  B.off_dxpart = take(DX_PART_BYTES);
  B.fixed = o;
  B.off_ghat_t = take(kept ? 0 : (size_t)S.Vp * Pw);
  B.off_gexp = take(kept ? 0 : (size_t)(S.Vp / 128) * (Pw / 128) * 4);      // block exponents of the dlogits
  B.part_stride = ((size_t)S.dq * S.Vp * 4 + 255) / 256 * 256;
  B.off_dwacc = take(B.part_stride * (size_t)nparts);     // fp32 dW partials, one per dW launch
  B.total = o;
  B.off_dwtail = o;
  B.tail_bytes = S.Np <= Pw ? dw_tail_plan(S.dq, S.Vp, S.Np).bytes : 0;       // (one dW launch over all rows, or no K-split)
  return B;
}

// Rows per panel: as many 256-row tiles as give the dX kernel one full round of tiles on the
// 256 CUs (its tile count is (P / 256) * (dq / 256)), capped by the problem size.
static int64_t default_panel(const SavedLayout& S) {
  int64_t rt = 256 / (S.dq / 256);
  if (rt < 1) rt = 1;
  if (rt > 64) rt = 64;
  const int64_t P = rt * 256;
  return S.Np < P ? S.Np : P;
}
// Rows per dW launch: several dX panels are gathered (transposed) before dW runs, so that its
// fp32 accumulator is read and rewritten less often and its K loop is long.
static int64_t default_dw_panel(const SavedLayout& S, int64_t P) {
  int64_t m = 131072 / P;
  if (m < 1) m = 1;
  int64_t Pw = m * P;
  const int64_t cap = round_up(S.Np, P);
  return Pw < cap ? Pw : cap;
}

// One fp32 dW partial per dW launch (plain stores, summed once at the end) as long as there are
// at most 8; beyond that the last buffer is read, added to and rewritten.
static int dw_launches(const SavedLayout& S, int64_t Pw) {
  const int64_t n = (S.Np + Pw - 1) / Pw;
  return (int)(n < 8 ? n : 8);
}

extern "C" int sce_version(void) { return SCE_VERSION; }

extern "C" int sce_timing_enable(int on) {
  std::lock_guard<std::mutex> lk(g_timing_mu);
  for (int k = 0; k < SCE_K_COUNT; ++k) {
    for (hipEvent_t e : g_timing.begin[k]) g_timing.pool.push_back(e);
    for (hipEvent_t e : g_timing.end[k]) g_timing.pool.push_back(e);
    g_timing.begin[k].clear(); g_timing.end[k].clear();
    g_timing.ms[k] = 0.0; g_timing.launches[k] = 0;
  }
  g_timing.on = on != 0;
  return SCE_OK;
}

extern "C" int sce_timing_read(sce_timing* out) {
  if (!out) return fail(SCE_EINVAL, "out is NULL");
  std::lock_guard<std::mutex> lk(g_timing_mu);
  for (int k = 0; k < SCE_K_COUNT; ++k) {
    const size_t n = g_timing.end[k].size();
    for (size_t i = 0; i < n; ++i) {
      float ms = 0.f;
      HIP_TRY(hipEventSynchronize(g_timing.end[k][i]));
      HIP_TRY(hipEventElapsedTime(&ms, g_timing.begin[k][i], g_timing.end[k][i]));
      g_timing.ms[k] += ms; g_timing.launches[k] += 1;
      g_timing.pool.push_back(g_timing.begin[k][i]); g_timing.pool.push_back(g_timing.end[k][i]);
    }
    g_timing.begin[k].clear(); g_timing.end[k].clear();
    out->ms[k] = g_timing.ms[k]; out->launches[k] = g_timing.launches[k];
  }
  return SCE_OK;
}
extern "C" const char* sce_last_error(void) { return g_err; }

// Forward splits V among S workgroups per row tile (each walks CT / S column tiles).  8 keeps the partial records
// small and gives every workgroup a long walk; more (up to 16) only where 8 would leave the last round of
// workgroups, one per CU, mostly empty.
constexpr int FWD_MAX_SPLITS = 16;
// SCE_FWD_KERNEL=pingpong in the environment selects the ping-pong walk (fwd_pp_kernel) for the dlogits-emitting
// forward pass.  It is complete and parity-tested, and on this part slower than fwd_kernel at every shape of the
// workload table (its 256 x 128 tiles are bound by L2 -> LDS traffic where K is long, and the vector ALU work of one
// wave delays the MFMAs of the other by about half its length where K is short), so it is not the default.
static bool fwd_pingpong_wanted() {
  const char* e = getenv("SCE_FWD_KERNEL");
  return e && strcmp(e, "pingpong") == 0;
}
static int fwd_splits(int RT, int CT, int ncu) {
  if (CT <= 8) return CT;
  auto fill = [&](int S) { const int64_t wg = (int64_t)RT * S; return (double)wg / (double)((wg + ncu - 1) / ncu * ncu); };
  int best = 8;
  for (int S = 9; S <= FWD_MAX_SPLITS && S <= CT; ++S)
    if (fill(S) > fill(best) + 0.03) best = S;
  return best;
}

extern "C" int sce_sizes_for(const sce_shape* shape, sce_sizes* out) {
  if (int rc = check_shape(shape)) return rc;
  if (!out) return fail(SCE_EINVAL, "out is NULL");
  const SavedLayout S = saved_layout(shape->N, shape->d, shape->V, shape->n_predict);
  out->saved_bytes = S.total;
  out->saved_x_bytes = S.x_total;
  out->wcache_bytes = S.w_total;
  out->fwd_workspace_bytes = (size_t)FWD_MAX_SPLITS * S.Np * 16 + 256;
  out->bwd_workspace_min_bytes = bwd_layout(S, 256, 256, 1, shape->n_predict).total;
  out->bwd_panel_rows = default_panel(S);
  {
    const int64_t Pw = default_dw_panel(S, out->bwd_panel_rows);
    // (both with room for the partial tiles of a K-split last round of dW, where there is to be one)
    const BwdLayout Bd = bwd_layout(S, out->bwd_panel_rows, Pw, dw_launches(S, Pw), shape->n_predict);
    out->bwd_workspace_bytes = Bd.total + Bd.tail_bytes;
    out->dlogits_bytes = S.g_total;
    const BwdLayout Bk = bwd_layout(S, out->bwd_panel_rows, Pw, dw_launches(S, Pw), shape->n_predict, true);
    out->bwd_workspace_kept_bytes = Bk.total + Bk.tail_bytes;
  }
  out->saved_bf16_bytes = saved_layout(shape->N, shape->d, shape->V, shape->n_predict, 2).total;
  return SCE_OK;
}

static int grid_for(size_t work_items, int per_block) {
  size_t g = (work_items + per_block - 1) / per_block;
  if (g > 65536 * 16) g = 65536 * 16;
  if (g == 0) g = 1;
  return (int)g;
}

static int quantize_impl(const void* src, int32_t src_dtype, void* dst, float inv_scale, const float* scale_dev, size_t n, int32_t device,
                         void* stream) {
  if (!src || !dst) return fail(SCE_EINVAL, "src/dst is NULL");
  if (int rc = check_device(device)) return rc;
  if (n == 0) return SCE_OK;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  hipStream_t st = (hipStream_t)stream;
  const int grid = grid_for((n + 3) / 4, 256);
  if (src_dtype == SCE_F32) quantize_flat_kernel<float><<<grid, 256, 0, st>>>((const float*)src, (uint8_t*)dst, n, inv_scale, scale_dev);
  else if (src_dtype == SCE_BF16) quantize_flat_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)src, (uint8_t*)dst, n, inv_scale, scale_dev);
  else return fail(SCE_EINVAL, "unsupported dtype %d", src_dtype);
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

extern "C" int sce_quantize_e4m3(const void* src, int32_t src_dtype, void* dst, double scale, size_t n, int32_t device,
                                 void* stream) {
  if (!(scale > 0.0)) return fail(SCE_EINVAL, "scale must be positive");
  return quantize_impl(src, src_dtype, dst, (float)(1.0 / scale), nullptr, n, device, stream);
}

extern "C" int sce_quantize_e4m3_dev(const void* src, int32_t src_dtype, void* dst, const float* scale_dev, size_t n, int32_t device,
                                     void* stream) {
  if (!scale_dev) return fail(SCE_EINVAL, "scale_dev is NULL");
  return quantize_impl(src, src_dtype, dst, 0.f, scale_dev, n, device, stream);
}

extern "C" int sce_amax_scale(const void* src, int32_t src_dtype, size_t n, float* scale_out, int32_t device, void* stream) {
  if (!src || !scale_out) return fail(SCE_EINVAL, "src/scale_out is NULL");
  if (n == 0) return fail(SCE_EINVAL, "n must be positive");
  if (src_dtype != SCE_F32 && src_dtype != SCE_BF16) return fail(SCE_EINVAL, "unsupported dtype %d", src_dtype);
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  hipStream_t st = (hipStream_t)stream;
  uint32_t* bits = reinterpret_cast<uint32_t*>(scale_out);
  int grid = grid_for(n, 256 * 16);
  if (grid > 4096) grid = 4096;
  amax_begin_kernel<<<1, 1, 0, st>>>(bits);
  if (src_dtype == SCE_F32) amax_kernel<float><<<grid, 256, 0, st>>>((const float*)src, n, bits);
  else amax_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)src, n, bits);
  amax_end_kernel<<<1, 1, 0, st>>>(bits);
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

extern "C" int sce_transpose_bytes(const void* src, void* dst, int64_t rows, int64_t cols, int32_t device, void* stream) {
  if (!src || !dst) return fail(SCE_EINVAL, "src/dst is NULL");
  if (rows <= 0 || cols <= 0) return fail(SCE_EINVAL, "rows and cols must be positive");
  if ((rows + 63) / 64 > 65535) return fail(SCE_EINVAL, "too many rows (%lld)", (long long)rows);
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  transpose_bytes_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)src, (uint8_t*)dst, rows, cols);
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

static int check_common(const sce_args* a) {
  if (!a) return fail(SCE_EINVAL, "args is NULL");
  if (a->struct_size != sizeof(sce_args)) return fail(SCE_EINVAL, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(sce_args));
  if (int rc = check_shape(&a->shape)) return rc;
  if (!a->targets) return fail(SCE_EINVAL, "targets is NULL");
  if (!(a->cap > 0.f) || a->cap > 40.f) return fail(SCE_EINVAL, "cap = %g must be in (0, 40]", (double)a->cap);
  if (a->operand_dtype == 0 && ((!a->x_s_dev && !(a->x_s > 0.0)) || (!a->w_s_dev && !(a->w_s > 0.0))))
    return fail(SCE_EINVAL, "x_s and w_s must be positive");
  if (a->reduction != SCE_REDUCE_NONE && a->reduction != SCE_REDUCE_MEAN) return fail(SCE_EINVAL, "bad reduction %d", a->reduction);
  if (!a->saved) return fail(SCE_EINVAL, "saved is NULL");
  if (((uintptr_t)a->saved & 255) || ((uintptr_t)a->workspace & 255) || ((uintptr_t)a->wcache & 255))
    return fail(SCE_EINVAL, "saved, workspace and wcache must be 256-byte aligned");
  if (a->vocab_limit < 0 || a->vocab_limit > a->shape.V) return fail(SCE_EINVAL, "vocab_limit must be in [0, V]");
  return check_device(a->device);
}

// ws: the partial records of the V-splits (the caller's workspace, or the library's static scratch)
static int forward_impl(const sce_args* a, void* ws, size_t ws_bytes, const char* ws_name) {
  const int64_t N = a->shape.N, d = a->shape.d, V = a->shape.V;
  if (!a->x || !a->w) return fail(SCE_EINVAL, "x or w is NULL");
  if (a->x_ld < d || a->w_ld < V) return fail(SCE_EINVAL, "row strides smaller than the row length");
  if (a->reduction == SCE_REDUCE_NONE && !a->losses) return fail(SCE_EINVAL, "losses is NULL with reduction = none");
  if (a->reduction == SCE_REDUCE_MEAN && !a->loss) return fail(SCE_EINVAL, "loss is NULL with reduction = mean");
  if (a->reduction == SCE_REDUCE_MEAN && a->shape.n_predict != 1)
    return fail(SCE_EINVAL, "reduction = mean is defined for a single offset only; use reduction = none with n_predict > 1");
  const bool bf16ops = a->operand_dtype == SCE_BF16;
  if (a->operand_dtype != 0 && !bf16ops) return fail(SCE_EINVAL, "operand_dtype %d: 0 (e4m3) or SCE_BF16", a->operand_dtype);
  if (bf16ops && (a->dlogits_from_forward || a->norm || a->wcache))
    return fail(SCE_EINVAL, "bf16 operands are for the forward-only eval head: no kept dlogits, fused norm or weight cache");
  const SavedLayout S = saved_layout(N, d, V, a->shape.n_predict, bf16ops ? 2 : 1);
  const size_t need_saved = a->wcache ? S.x_total : S.total;
  if (a->saved_bytes < need_saved) return fail(SCE_EINVAL, "saved buffer too small: %zu < %zu", a->saved_bytes, need_saved);
  if (a->wcache && a->wcache_bytes < S.w_total) return fail(SCE_EINVAL, "weight cache too small: %zu < %zu", a->wcache_bytes, S.w_total);
  const int64_t Vl = a->vocab_limit > 0 ? a->vocab_limit : V;       // columns that take part
  const int RT = (int)(S.Np / 256), CT = (int)((Vl + 255) / 256);
  const size_t gneed = need_saved + (a->dlogits_from_forward ? S.g_total : 0);
  if (a->saved_bytes < gneed) return fail(SCE_EINVAL, "saved buffer too small for the dlogits: %zu < %zu", a->saved_bytes, gneed);
  DeviceGuard guard(a->device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", a->device);
  (void)hipGetLastError();          // an error left by some earlier, unrelated call is not this call's
  hipStream_t st = (hipStream_t)a->stream;
  uint8_t* sv = (uint8_t*)a->saved;
  uint8_t* xq = sv + S.off_xq;
  uint8_t* wbase = a->wcache ? (uint8_t*)a->wcache : sv + S.x_total;
  uint8_t* wqt = wbase + S.rel_wqt;
  uint8_t* wq = wbase + S.rel_wq;
  uint8_t* gbase = sv + need_saved;       // dlogits, when the forward pass emits them

  // a scale that lives on the device: its value and what follows from it go into the header of `saved`, for the
  // kernels of this call and of the matching backward
  const bool devsc = a->x_s_dev || a->w_s_dev;
  DevConsts* dcp = devsc ? (DevConsts*)(sv + S.off_hdr + 32) : nullptr;
  const float inv_xs = a->x_s_dev ? 0.f : (float)(1.0 / a->x_s), inv_ws = a->w_s_dev ? 0.f : (float)(1.0 / a->w_s);
  {
    KernelTimer tm(SCE_K_QUANT, st);
    if (bf16ops) {
      const int grid = grid_for((size_t)S.Np * (S.dp / 16), 256);
      if (a->x_dtype == SCE_F32) prep_x_bf16_kernel<float><<<grid, 256, 0, st>>>((const float*)a->x, a->x_ld, N, d, (uint16_t*)xq, S.Np, S.dp / 2, S.ldx / 2);
      else if (a->x_dtype == SCE_BF16) prep_x_bf16_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)a->x, a->x_ld, N, d, (uint16_t*)xq, S.Np, S.dp / 2, S.ldx / 2);
      else return fail(SCE_EINVAL, "unsupported x dtype %d", a->x_dtype);
      dim3 gw((unsigned)(S.Vp / 64), (unsigned)(S.dp / 2 / 64));
      if (a->w_dtype == SCE_F32) prep_w_bf16_kernel<float><<<gw, 256, 0, st>>>((const float*)a->w, a->w_ld, d, V, (uint16_t*)wqt, S.ldx / 2);
      else if (a->w_dtype == SCE_BF16) prep_w_bf16_kernel<bf16_t><<<gw, 256, 0, st>>>((const bf16_t*)a->w, a->w_ld, d, V, (uint16_t*)wqt, S.ldx / 2);
      else return fail(SCE_EINVAL, "unsupported w dtype %d", a->w_dtype);
    }
    if (devsc && !bf16ops) dev_consts_kernel<<<1, 1, 0, st>>>(a->x_s_dev, a->w_s_dev, (float)a->x_s, (float)a->w_s, a->cap, dcp);
    const int grid = grid_for((size_t)S.Np * (S.dp / 16), 256);
    float* rstd = (float*)(sv + S.off_rstd);
    const int ngrid = (int)((S.Np + 3) / 4);
    if (bf16ops) {
      // operands laid out above
    } else if (a->norm && a->x_dtype == SCE_F32)
      rmsnorm_quantize_kernel<float><<<ngrid, 256, 0, st>>>((const float*)a->x, a->x_ld, N, d, a->norm_eps, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev, rstd);
    else if (a->norm && a->x_dtype == SCE_BF16)
      rmsnorm_quantize_kernel<bf16_t><<<ngrid, 256, 0, st>>>((const bf16_t*)a->x, a->x_ld, N, d, a->norm_eps, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev, rstd);
    else if (a->x_dtype == SCE_F32)
      quantize_pad_kernel<float><<<grid, 256, 0, st>>>((const float*)a->x, a->x_ld, N, d, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev);
    else if (a->x_dtype == SCE_BF16)
      quantize_pad_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)a->x, a->x_ld, N, d, xq, S.Np, S.dp, S.ldx, inv_xs, a->x_s_dev);
    else return fail(SCE_EINVAL, "unsupported x dtype %d", a->x_dtype);
    dim3 gw((unsigned)(S.Vp / 64), (unsigned)(S.dq / 64));
    if (bf16ops) {
    } else if (a->wcache && a->wcache_valid) {
      // the caller vouches that the cache holds e4m3(W / w_s) of this W (unchanged since an earlier call)
    } else if (a->w_dtype == SCE_F32)
      quantize_w_kernel<float><<<gw, 256, 0, st>>>((const float*)a->w, a->w_ld, d, V, wq, wqt, S.dp, S.ldx, S.Vp / BK, inv_ws, a->w_s_dev);
    else if (a->w_dtype == SCE_BF16)
      quantize_w_kernel<bf16_t><<<gw, 256, 0, st>>>((const bf16_t*)a->w, a->w_ld, d, V, wq, wqt, S.dp, S.ldx, S.Vp / BK, inv_ws, a->w_s_dev);
    else return fail(SCE_EINVAL, "unsupported w dtype %d", a->w_dtype);
  }
  const bool emit = a->dlogits_from_forward != 0;
  const int CTw = emit ? (int)(S.Vp / 256) : CT;       // with the dlogits every tile is visited: the masked ones must read as zero later
  const int nsplit = fwd_splits(RT, CTw, device_cus_or_default(a->device));
  const size_t need_ws = (size_t)nsplit * S.Np * 16;
  if (!ws || ws_bytes < need_ws) return fail(SCE_EINVAL, "%s too small: %zu < %zu", ws_name, ws_bytes, need_ws);
  FwdParams p;
  p.xq = xq; p.wqt = wqt; p.partials = (float4*)ws;
  p.targets = a->targets; p.ignore_index = a->ignore_index; p.n_predict = a->shape.n_predict; p.s_uy = (float*)(sv + S.off_zy);
  p.ghat_t = emit ? gbase + S.rel_g : nullptr; p.gexp = emit ? (uint32_t*)(gbase + S.rel_gexp) : nullptr; p.kbw = S.Np / BK;
  p.dp = S.dp; p.ldx = S.ldx; p.N = (int)N; p.V = (int)Vl; p.Np = (int)S.Np; p.RT = RT; p.CT = CTw; p.S = nsplit;
  p.sc = bf16ops ? 1.0f : (float)a->x_s * (float)a->w_s; p.k1 = p.sc * 2.0f * LOG2E / a->cap; p.c2 = -2.0f * a->cap * LOG2E; p.ic2 = 1.0f / p.c2;
  p.dc = bf16ops ? nullptr : dcp;
  p.want_argmax = a->argmax != nullptr;
  const int grid = 8 * nsplit * ((RT + 7) / 8);
  {
    // the exponent boosts of the rows, from the tile in the middle of the vocabulary (kept for backward in either mode)
    KernelTimer tm(SCE_K_QUANT, st);
    float* lam = (float*)(sv + S.off_lam);
    p.lam = lam;
    if (!bf16ops) fwd_sample_kernel<<<RT, NTHREADS, SMEM_BYTES, st>>>(p, CT / 2, lam);
  }
  {
    KernelTimer tm(SCE_K_FWD, st);
    if (emit && fwd_pingpong_wanted()) {
      // (all tile loads are issued by the accumulating waves: measured faster than sharing them out, and a wait that the
      // compiler adds in an epilogue unit then has no tile load to wait for)
      if (a->argmax) fwd_pp_kernel<12, true><<<grid, PP_THREADS, SMEM_FWD_PP, st>>>(p);
      else fwd_pp_kernel<12, false><<<grid, PP_THREADS, SMEM_FWD_PP, st>>>(p);
    } else if (emit) fwd_kernel<true><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
    else if (bf16ops) fwd_kernel<false, true><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
    else fwd_kernel<false><<<grid, NTHREADS, SMEM_FWD, st>>>(p);
  }
  KernelTimer tm_red(SCE_K_FWD_REDUCE, st);
  float* s_lse = (float*)(sv + S.off_lse);
  float* s_umax = (float*)(sv + S.off_umax);
  float* s_zy = (float*)(sv + S.off_zy);
  fwd_combine_kernel<<<(int)(S.Np / 256), 256, 0, st>>>(p.partials, nsplit, (int)N, (int)S.Np, (int)Vl, a->targets, a->ignore_index,
                                                       a->cap, a->mtp_weights, a->shape.n_predict, s_lse, s_umax, s_zy, a->losses, a->lse,
                                                       a->argmax);
  fwd_reduce_kernel<<<1, 1024, 0, st>>>(p.partials, (int)(S.Np / 256), (int32_t*)(sv + S.off_hdr),
                                        a->reduction == SCE_REDUCE_MEAN ? a->loss : nullptr, a->n_valid);
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

extern "C" int sce_forward(const sce_args* a) {
  if (int rc = check_common(a)) return rc;
  return forward_impl(a, a->workspace, a->workspace_bytes, "forward workspace");
}

// The same launches as sce_forward with the partial records in the library's static device array instead of a
// caller's workspace: no allocation, by the caller for this call or by the library ever.  Calls on one device share
// the array; nothing in it has to start at zero (the forward kernel writes every record that the combine kernel
// reads), so nothing is cleared, but two calls in flight on one device at a time would overwrite each other's records.
extern "C" int sce_forward_noalloc(const sce_args* a) {
  if (int rc = check_common(a)) return rc;
  void* sp = g_scratch[a->device];              // set by check_device (inside check_common) for this very device
  if (!sp) return fail(SCE_EHIP, "no static scratch on device %d", a->device);
  return forward_impl(a, sp, NOALLOC_SCRATCH_BYTES,
                      "the static scratch of sce_forward_noalloc (8 MiB: N rounded up to 256 times the number of V-splits, 8 to 16, "
                      "may not exceed 524288; use sce_forward with a workspace)");
}

extern "C" int sce_backward(const sce_args* a) {
  if (int rc = check_common(a)) return rc;
  const int64_t N = a->shape.N, d = a->shape.d, V = a->shape.V;
  if (a->operand_dtype != 0) return fail(SCE_EINVAL, "bf16 operands are forward only (the eval head)");
  if (!a->grad_output) return fail(SCE_EINVAL, "grad_output is NULL");
  if (!a->dx || !a->dw) return fail(SCE_EINVAL, "dx or dw is NULL");
  if (a->norm) {
    if (!a->x) return fail(SCE_EINVAL, "norm is set: backward needs x (the hidden state given to forward)");
    if (a->x_dtype != SCE_F32 && a->x_dtype != SCE_BF16) return fail(SCE_EINVAL, "unsupported x dtype %d", a->x_dtype);
    if (a->x_ld < d) return fail(SCE_EINVAL, "row strides smaller than the row length");
  }
  if (a->dx_ld < d || a->dw_ld < V) return fail(SCE_EINVAL, "row strides smaller than the row length");
  if ((a->dx_dtype != SCE_F32 && a->dx_dtype != SCE_BF16) || (a->dw_dtype != SCE_F32 && a->dw_dtype != SCE_BF16))
    return fail(SCE_EINVAL, "unsupported gradient dtype");
  const SavedLayout S = saved_layout(N, d, V, a->shape.n_predict);
  const size_t need_saved = a->wcache ? S.x_total : S.total;
  if (a->saved_bytes < need_saved) return fail(SCE_EINVAL, "saved buffer too small: %zu < %zu", a->saved_bytes, need_saved);
  if (a->wcache && a->wcache_bytes < S.w_total) return fail(SCE_EINVAL, "weight cache too small: %zu < %zu", a->wcache_bytes, S.w_total);
  const int64_t Vl = a->vocab_limit > 0 ? a->vocab_limit : V;       // columns that take part
  if (!a->workspace) return fail(SCE_EINVAL, "workspace is NULL");
  const int K = a->shape.n_predict;
  const bool kept = a->dlogits_from_forward != 0;        // the dlogits came with `saved`
  if (kept && a->saved_bytes < need_saved + S.g_total)
    return fail(SCE_EINVAL, "saved buffer too small for the dlogits: %zu < %zu", a->saved_bytes, need_saved + S.g_total);
  const BwdLayout Bmin = bwd_layout(S, 256, 256, 1, K, kept);
  if (a->workspace_bytes < Bmin.total) return fail(SCE_EINVAL, "backward workspace too small: %zu < %zu", a->workspace_bytes, Bmin.total);
  if (a->panel_rows % 256) return fail(SCE_EINVAL, "panel_rows must be a multiple of 256");
  // panel sizes from what the caller gave: P rows per recompute/dX panel, Pw = m * P rows per dW launch
  int64_t P, Pw;
  int nparts;
  if (kept) {
    // dX still goes panel by panel, one round of tiles each: a launch with several rounds was measured 2 % slower
    P = a->panel_rows > 0 ? a->panel_rows : default_panel(S);
    if (P > S.Np) P = S.Np;
    if (P > 131072) P = 131072;
    Pw = default_dw_panel(S, P);
    nparts = dw_launches(S, Pw);
    while (nparts > 1 && bwd_layout(S, P, Pw, nparts, K, true).total > a->workspace_bytes) --nparts;
  } else {
    // bytes left for the e4m3 dlogits: Vp rows of Pw bytes
    const int64_t room = (int64_t)(a->workspace_bytes - Bmin.fixed - Bmin.part_stride);
    P = default_panel(S);
    if (a->panel_rows > 0) {
      P = a->panel_rows < S.Np ? a->panel_rows : S.Np;
      if (P > 131072) P = 131072;          // a dW launch covers at least one panel and at most MAX_SCALE_KBLOCKS K blocks
    }
    if (P * S.Vp > room) P = room / S.Vp / 256 * 256;
    if (P < 256) P = 256;                                  // Bmin fits, as checked above
    Pw = default_dw_panel(S, P);
    if (Pw * S.Vp > room) Pw = room / S.Vp / P * P;
    if (Pw < P) Pw = P;
    nparts = dw_launches(S, Pw);
    // the estimate above ignores the 256-byte alignment of each region: settle on a layout that fits
    while (bwd_layout(S, P, Pw, nparts, K).total > a->workspace_bytes) {
      if (nparts > 1) --nparts;
      else if (Pw > P) Pw -= P;
      else if (P > 256) { P -= 256; Pw = P; }
      else return fail(SCE_EINVAL, "internal: panel layout exceeds workspace");
    }
  }
  const BwdLayout B = bwd_layout(S, P, Pw, nparts, K, kept);
  DeviceGuard guard(a->device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", a->device);
  (void)hipGetLastError();          // an error left by some earlier, unrelated call is not this call's
  hipStream_t st = (hipStream_t)a->stream;
  uint8_t* sv = (uint8_t*)a->saved;
  uint8_t* ws = (uint8_t*)a->workspace;
  const uint8_t* xq = sv + S.off_xq;
  const uint8_t* wbase = a->wcache ? (const uint8_t*)a->wcache : sv + S.x_total;
  const uint8_t* wqt = wbase + S.rel_wqt;
  const uint8_t* wq = wbase + S.rel_wq;
  const float* s_lse = (const float*)(sv + S.off_lse);
  const float* s_zy = (const float*)(sv + S.off_zy);
  const int32_t* hdr = (const int32_t*)(sv + S.off_hdr);
  const DevConsts* dcp = (a->x_s_dev || a->w_s_dev) ? (const DevConsts*)(sv + S.off_hdr + 32) : nullptr;     // as forward left it
  uint8_t* gkept = sv + need_saved;
  uint32_t* gexp = kept ? (uint32_t*)(gkept + S.rel_gexp) : (uint32_t*)(ws + B.off_gexp);
  float* rho = (float*)(ws + B.off_rho);
  int32_t* rowinfo = (int32_t*)(ws + B.off_rowinfo);
  float* hcoef = (float*)(ws + B.off_hcoef);
  float* blockmax = (float*)(ws + B.off_blockmax);
  float* xi = (float*)(ws + B.off_xi);
  uint8_t* xt = ws + B.off_xt;
  float* dwacc = (float*)(ws + B.off_dwacc);
  int32_t* perm = (int32_t*)(ws + B.off_perm);
  const int64_t NE = N * K;            // one-hot entries: one per (offset, row)
  int32_t* vals_in = perm + NE;
  int32_t* skeys = (int32_t*)(ws + B.off_keys);
  int32_t* keys_in = skeys + NE;
  int32_t* segoff = (int32_t*)(ws + B.off_segoff);
  int32_t* longlist = (int32_t*)(ws + B.off_longlist);
  float* longsum = (float*)(ws + B.off_longsum);
  int32_t* longbase = (int32_t*)(ws + B.off_longbase);
  uint8_t* ghat_t = kept ? gkept + S.rel_g : ws + B.off_ghat_t;
  const int64_t gkb = kept ? S.Np / BK : Pw / BK;      // K blocks per v tile of the dlogits buffer

  const int nblk = (int)(S.Np / 256);
  KernelTimer* tm_prep = new KernelTimer(SCE_K_BWD_PREP, st);
  bwd_prep_kernel<<<nblk, 256, 0, st>>>(s_lse, s_zy, a->targets, a->ignore_index, hdr, a->grad_output,
                                        a->reduction == SCE_REDUCE_NONE ? 1 : 0, a->grad_scale, a->mtp_weights, K, a->cap, (int)N,
                                        (int)S.Np, (int)Vl, (const float*)(sv + S.off_lam), rho, hcoef, blockmax, kept ? nullptr : rowinfo);
  bwd_xi_kernel<<<1, 1024, 0, st>>>(blockmax, nblk, xi);
  {
    dim3 g((unsigned)(S.Np / 64), (unsigned)(S.dq / 64));
    bwd_xt_kernel<<<g, 256, 0, st>>>(xq, S.dp, S.ldx, S.Np / BK, rho, xi, xt);
  }
  // rows grouped by target, for the one-hot part of dW
  {
    bwd_keys_kernel<<<(int)((NE + 255) / 256), 256, 0, st>>>(a->targets, a->ignore_index, (int)N, (int)S.Np, (int)Vl, (int)V, K, keys_in, vals_in, longlist);
    int bits = 1;
    while ((1ll << bits) <= V) ++bits;
    size_t tmp = B.sorttmp_bytes;
    if (sce::sort_pairs(ws + B.off_sorttmp, &tmp, keys_in, skeys, vals_in, perm, (size_t)NE, bits, st) != 0)
    { delete tm_prep; return fail(SCE_EHIP, "radix sort of the targets failed"); }
    bwd_segoff_kernel<<<(int)((NE + 256) / 256), 256, 0, st>>>(skeys, (int)NE, (int)V, segoff);
    bwd_longlist_kernel<<<(int)((V + 255) / 256), 256, 0, st>>>(segoff, (int)V, longlist, longbase);
  }
  delete tm_prep;
  const float k1 = (float)a->x_s * (float)a->w_s * 2.0f * LOG2E / a->cap, c2 = -2.0f * a->cap * LOG2E;
  const int CTv = (int)(S.Vp / 256), CTd = (int)(S.dq / 256);
  int launch = 0;
  DwTail tail;
  tail.buf = nullptr; tail.tile0 = -1; tail.ntail = 0; tail.kp = 1; tail.share = 1;
  int64_t w0 = 0;                      // first row of the rows gathered for the next dW launch
  for (int64_t p0 = 0; p0 < S.Np; p0 += P) {
    const int64_t prow = (S.Np - p0 < P) ? (S.Np - p0) : P;     // multiple of 256
    const int RTp = (int)(prow / 256);
    const int64_t gorg = kept ? 0 : w0;                         // the row that K block 0 of the dlogits buffer stands for
    if (!kept) {
      RecomputeParams rp;
      rp.xq = xq + p0 * S.ldx; rp.wqt = wqt; rp.ghat_t = ghat_t; rp.gexp = gexp; rp.rowinfo = rowinfo + p0; rp.Np = S.Np; rp.n_predict = K;
      rp.dp = S.dp; rp.ldx = S.ldx; rp.kbw = gkb; rp.kb0 = (p0 - gorg) / BK; rp.RT = RTp; rp.CT = CTv; rp.V = (int)Vl; rp.k1 = k1; rp.c2 = c2; rp.dc = dcp;
      {
        KernelTimer tm(SCE_K_RECOMPUTE, st);
        bwd_recompute_kernel<<<map_tile_grid(RTp, CTv), NTHREADS, SMEM_RECOMPUTE, st>>>(rp);
      }
    }

    DxParams dp_;
    dp_.wq = wq; dp_.ghat_t = ghat_t + ((p0 - gorg) / BK) * BLOCKED_KSTEP; dp_.gexp = gexp + (p0 - gorg) / BK; dp_.kbw = gkb; dp_.wqt = wqt; dp_.rho = rho + p0; dp_.hcoef = hcoef + p0; dp_.targets = a->targets + p0;
    dp_.dx_ld = a->dx_ld; dp_.Vp = S.Vp; dp_.ldx = S.ldx; dp_.Np = S.Np; dp_.dq = S.dq; dp_.RT = RTp; dp_.CT = CTd;
    dp_.n_predict = K; dp_.rows_left = (int)(N - p0 > 0 ? N - p0 : 0);
    dp_.rows = (int)((N - p0 < prow) ? (N - p0 > 0 ? N - p0 : 0) : prow); dp_.d = (int)d; dp_.V = (int)Vl; dp_.w_s = (float)a->w_s; dp_.dc = dcp;
    dp_.part = (float*)(ws + B.off_dxpart);
    // a panel with fewer than half as many tiles as there are CUs shares each tile's K loop among several workgroups
    const int tiles = RTp * CTd, kpairs = (int)(S.Vp / BK / 2);
    int ksplit = tiles * 2 <= 256 ? 256 / tiles : 1;
    if (ksplit > 8) ksplit = 8;
    if (ksplit > kpairs) ksplit = kpairs;
    dp_.ksplit = ksplit;
    {
      KernelTimer tm(SCE_K_DX, st);
      const bool f32 = a->dx_dtype == SCE_F32;
      const int smem_dx = smem_scaled((int)(S.Vp / BK), SMEM_DX);
      dp_.dx = f32 ? (void*)((float*)a->dx + p0 * a->dx_ld) : (void*)((bf16_t*)a->dx + p0 * a->dx_ld);
      if (ksplit == 1) {
        if (f32) bwd_dx_kernel<float, false><<<map_tile_grid(RTp, CTd), NTHREADS, smem_dx, st>>>(dp_);
        else bwd_dx_kernel<bf16_t, false><<<map_tile_grid(RTp, CTd), NTHREADS, smem_dx, st>>>(dp_);
      } else if (dp_.rows > 0) {
        const int fgrid = (int)(((int64_t)dp_.rows * (d / 4) + 255) / 256);
        if (f32) {
          bwd_dx_kernel<float, true><<<map_tile_grid(RTp, CTd * ksplit), NTHREADS, smem_dx, st>>>(dp_);
          bwd_dx_finish_kernel<float><<<fgrid, 256, 0, st>>>(dp_);
        } else {
          bwd_dx_kernel<bf16_t, true><<<map_tile_grid(RTp, CTd * ksplit), NTHREADS, smem_dx, st>>>(dp_);
          bwd_dx_finish_kernel<bf16_t><<<fgrid, 256, 0, st>>>(dp_);
        }
      }
    }

    const int64_t gathered = p0 + prow - w0;
    if (gathered + P > Pw || p0 + prow >= S.Np) {      // the transposed scratch is full, or this was the last panel
      DwParams wp;
      const int part = launch < nparts ? launch : nparts - 1;
      wp.xt = xt; wp.ghat_t = ghat_t + ((w0 - gorg) / BK) * BLOCKED_KSTEP; wp.gexp = gexp + (w0 - gorg) / BK; wp.dwacc = (float*)((uint8_t*)dwacc + (size_t)part * B.part_stride);
      wp.kbn = S.Np / BK; wp.kbw = gkb; wp.kb0 = w0 / BK; wp.Vp = S.Vp;
      wp.RT = CTd; wp.CT = CTv; wp.KT = (int)(gathered / BK);
      {
        KernelTimer tm(SCE_K_DW, st);
        // When this launch is the only one and its last round of tiles would leave many CUs idle, that round is
        // shared out along K instead (bwd_dw_tail_kernel): the full rounds run as they are.
        const DwTailPlan tp = dw_tail_plan(S.dq, S.Vp, gathered);
        const bool only = w0 == 0 && p0 + prow >= S.Np && launch == 0;
        if (only && tp.use && B.tail_bytes >= tp.bytes && a->workspace_bytes >= B.off_dwtail + tp.bytes) {
          const int full = tp.full;
          tail.buf = (float*)(ws + B.off_dwtail); tail.tile0 = tp.full; tail.ntail = tp.ntail; tail.kp = tp.kp; tail.share = tp.share;
          if (full > 0) bwd_dw_kernel<false><<<full, NTHREADS, smem_scaled(wp.KT, 0), st>>>(wp);
          bwd_dw_tail_kernel<<<DW_TAIL_WGS, NTHREADS, smem_scaled(2 * tp.share, 0), st>>>(wp, tail);
        } else if (launch >= nparts) bwd_dw_kernel<true><<<map_tile_rr_grid(CTd, CTv), NTHREADS, smem_scaled(wp.KT, 0), st>>>(wp);
        else bwd_dw_kernel<false><<<map_tile_rr_grid(CTd, CTv), NTHREADS, smem_scaled(wp.KT, 0), st>>>(wp);
      }
      ++launch;
      w0 = p0 + prow;
    }
  }
  if (a->norm) {       // dX so far is the gradient of the normalised rows: take it through the norm, in place
    const float* rstd = (const float*)(sv + S.off_rstd);
    const int ngrid = (int)((N + 3) / 4);
    const bool gf = a->dx_dtype == SCE_F32, hf = a->x_dtype == SCE_F32;
    if (gf && hf) rmsnorm_backward_kernel<float, float><<<ngrid, 256, 0, st>>>((float*)a->dx, a->dx_ld, (const float*)a->x, a->x_ld, rstd, N, d);
    else if (gf) rmsnorm_backward_kernel<float, bf16_t><<<ngrid, 256, 0, st>>>((float*)a->dx, a->dx_ld, (const bf16_t*)a->x, a->x_ld, rstd, N, d);
    else if (hf) rmsnorm_backward_kernel<bf16_t, float><<<ngrid, 256, 0, st>>>((bf16_t*)a->dx, a->dx_ld, (const float*)a->x, a->x_ld, rstd, N, d);
    else rmsnorm_backward_kernel<bf16_t, bf16_t><<<ngrid, 256, 0, st>>>((bf16_t*)a->dx, a->dx_ld, (const bf16_t*)a->x, a->x_ld, rstd, N, d);
  }
  KernelTimer tm_fin(SCE_K_DW_FINAL, st);
  bwd_dw_long_kernel<<<dim3((unsigned)(NE / LONG_SEG + 1), (unsigned)(S.dq / 256)), 256, 0, st>>>(longlist, segoff, perm, hcoef, xq, S.dp, S.ldx, S.dq, (int)S.Np, longsum);
  {
    dim3 g((unsigned)((V + 63) / 64), (unsigned)((d + 63) / 64));
    if (a->dw_dtype == SCE_F32)
      bwd_dw_final_kernel<float><<<g, 256, 0, st>>>(dwacc, launch < nparts ? launch : nparts, (int64_t)(B.part_stride / 4), S.Vp, segoff, perm, hcoef, xq, S.ldx, (int)S.Np, xi, longsum, longbase, S.dq, (float)a->x_s, dcp, (int)d, (int)V,
                                                   (float*)a->dw, a->dw_ld, tail, CTd, CTv);
    else
      bwd_dw_final_kernel<bf16_t><<<g, 256, 0, st>>>(dwacc, launch < nparts ? launch : nparts, (int64_t)(B.part_stride / 4), S.Vp, segoff, perm, hcoef, xq, S.ldx, (int)S.Np, xi, longsum, longbase, S.dq, (float)a->x_s, dcp, (int)d, (int)V,
                                                    (bf16_t*)a->dw, a->dw_ld, tail, CTd, CTv);
  }
  HIP_TRY(hipGetLastError());
  return SCE_OK;
}

// ------------------------------------------------------------------------------------------
// measurement aids
// ------------------------------------------------------------------------------------------
static double median_mhz(const long long* clk, int n) {
  std::vector<double> v;
  for (int i = 0; i < n; ++i)
    if (clk[2 * i + 1] > 0) v.push_back((double)clk[2 * i] / (double)clk[2 * i + 1] * 100.0);
  if (v.empty()) return 0.0;
  std::sort(v.begin(), v.end());
  return v[v.size() / 2];
}

extern "C" int sce_bench_mfma(const void* random_bytes, int32_t iters, int32_t reps, void* scratch, size_t scratch_bytes, int32_t device,
                              void* stream, double* tflops, double* shader_mhz) {
  if (!scratch || !tflops || !shader_mhz || iters <= 0 || reps <= 0) return fail(SCE_EINVAL, "bad argument");
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  const int ncu = device_cus_or_default(device), grid = 4 * ncu;           // one wave per SIMD would be grid = ncu; four keep every SIMD fed
  const size_t need = (size_t)grid * 256 * 4 + 2 * 1024 * sizeof(long long);
  if (scratch_bytes < need) return fail(SCE_EINVAL, "scratch too small: %zu < %zu", scratch_bytes, need);
  hipStream_t st = (hipStream_t)stream;
  float* out = (float*)scratch;
  long long* clk = (long long*)((uint8_t*)scratch + (size_t)grid * 256 * 4);
  hipEvent_t e0, e1;
  HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
  bench_mfma_kernel<<<grid, 256, 0, st>>>((const uint8_t*)random_bytes, iters, out, clk);      // warm-up
  HIP_TRY(hipEventRecord(e0, st));
  for (int r = 0; r < reps; ++r) bench_mfma_kernel<<<grid, 256, 0, st>>>((const uint8_t*)random_bytes, iters, out, clk);
  HIP_TRY(hipEventRecord(e1, st));
  HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  std::vector<long long> h(2 * 1024);
  HIP_TRY(hipMemcpy(h.data(), clk, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
  (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
  const double flops = (double)reps * grid * 4.0 * iters * 16.0 * (2.0 * 32 * 32 * 64);
  *tflops = flops / (ms * 1e-3) * 1e-12;
  *shader_mhz = median_mhz(h.data(), grid < 1024 ? grid : 1024);
  return SCE_OK;
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

extern "C" int sce_bench_pingpong(const void* A, const void* B, int64_t M, int64_t N, int64_t K, int32_t valu_copies, int32_t reps, void* scratch,
                                  size_t scratch_bytes, int32_t device, void* stream, double* ms_per_launch) {
  if (!A || !B || !scratch || !ms_per_launch || reps <= 0) return fail(SCE_EINVAL, "bad argument");
  if (M <= 0 || N <= 0 || K <= 0 || M % 256 || N % 256 || K % 256 || M < 2048) return fail(SCE_EINVAL, "M, N, K must be positive multiples of 256, M at least 2048");
  if (valu_copies < 0 || valu_copies > 3) return fail(SCE_EINVAL, "valu_copies must be 0..3");
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  const int RT = (int)(N / 256), CT2 = (int)(M / 128), grid = map_tile_grid(RT, 8);
  if (scratch_bytes < (size_t)grid * PP_THREADS * 4) return fail(SCE_EINVAL, "scratch too small: %zu < %zu", scratch_bytes, (size_t)grid * PP_THREADS * 4);
  hipStream_t st = (hipStream_t)stream;
  const int64_t ld = row_stride(K);
  const int KD = (int)(K / BK);
  auto launch = [&]() {
    const uint8_t* a = (const uint8_t*)A; const uint8_t* b = (const uint8_t*)B; float* c = (float*)scratch;
    switch (valu_copies) {
      case 0: bench_pp_kernel<0><<<grid, PP_THREADS, PP_RING, st>>>(a, b, c, KD, RT, CT2, ld); break;
      case 1: bench_pp_kernel<1><<<grid, PP_THREADS, PP_RING, st>>>(a, b, c, KD, RT, CT2, ld); break;
      case 2: bench_pp_kernel<2><<<grid, PP_THREADS, PP_RING, st>>>(a, b, c, KD, RT, CT2, ld); break;
      default: bench_pp_kernel<3><<<grid, PP_THREADS, PP_RING, st>>>(a, b, c, KD, RT, CT2, ld); break;
    }
  };
  HIP_TRY(hipFuncSetAttribute((const void*)bench_pp_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize, PP_RING));
  HIP_TRY(hipFuncSetAttribute((const void*)bench_pp_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, PP_RING));
  HIP_TRY(hipFuncSetAttribute((const void*)bench_pp_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, PP_RING));
  HIP_TRY(hipFuncSetAttribute((const void*)bench_pp_kernel<3>, hipFuncAttributeMaxDynamicSharedMemorySize, PP_RING));
  hipEvent_t e0, e1;
  HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
  launch();
  HIP_TRY(hipEventRecord(e0, st));
  for (int r = 0; r < reps; ++r) launch();
  HIP_TRY(hipEventRecord(e1, st));
  HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
  HIP_TRY(hipGetLastError());
  *ms_per_launch = ms / reps;
  return SCE_OK;
}

extern "C" int sce_bench_gemm(const void* A, const void* B, int64_t M, int64_t N, int64_t K, int32_t reps, void* scratch, size_t scratch_bytes,
                              int32_t device, void* stream, double* tflops, double* shader_mhz) {
  if (!A || !B || !scratch || !tflops || !shader_mhz || reps <= 0) return fail(SCE_EINVAL, "bad argument");
  if (M <= 0 || N <= 0 || K <= 0 || M % 256 || N % 256 || K % 256) return fail(SCE_EINVAL, "M, N, K must be positive multiples of 256");
  if (int rc = check_device(device)) return rc;
  DeviceGuard guard(device);
  if (!guard.ok) return fail(SCE_EHIP, "cannot select device %d", device);
  const int RT = (int)(M / 256), CT = (int)(N / 256), grid = map_tile_grid(RT, CT);
  const size_t need = (size_t)grid * 256 * 4 + 2 * 1024 * sizeof(long long);
  if (scratch_bytes < need) return fail(SCE_EINVAL, "scratch too small: %zu < %zu", scratch_bytes, need);
  HIP_TRY(hipFuncSetAttribute((const void*)bench_gemm_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES));
  hipStream_t st = (hipStream_t)stream;
  float* out = (float*)scratch;
  long long* clk = (long long*)((uint8_t*)scratch + (size_t)grid * 256 * 4);
  const int64_t ld = row_stride(K);
  hipEvent_t e0, e1;
  HIP_TRY(hipEventCreate(&e0)); HIP_TRY(hipEventCreate(&e1));
  bench_gemm_kernel<<<grid, NTHREADS, SMEM_BYTES, st>>>((const uint8_t*)A, (const uint8_t*)B, out, (int)(K / BK), RT, CT, ld, clk);
  HIP_TRY(hipEventRecord(e0, st));
  for (int r = 0; r < reps; ++r)
    bench_gemm_kernel<<<grid, NTHREADS, SMEM_BYTES, st>>>((const uint8_t*)A, (const uint8_t*)B, out, (int)(K / BK), RT, CT, ld, clk);
  HIP_TRY(hipEventRecord(e1, st));
  HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  std::vector<long long> h(2 * 1024);
  HIP_TRY(hipMemcpy(h.data(), clk, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
  (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
  *tflops = 2.0 * M * N * K * reps / (ms * 1e-3) * 1e-12;
  *shader_mhz = median_mhz(h.data(), grid < 1024 ? grid : 1024);
  return SCE_OK;
}
