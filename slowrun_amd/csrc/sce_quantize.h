// Quantisation kernels: X and W to padded e4m3 operand arrays (with the final RMSNorm fused on request), amax scales,
// the bf16 operands of the eval head, byte transposes (internal header).
// Part of the one translation unit sce_kernels.hip, which includes it after the headers it builds on.
#pragma once

namespace sce {

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

// W (d, V) -> W_q (dq rows, K = Vp, tile by tile) and W_q^T [Vp][dp] (row-major); 128 x 128 tiles through LDS, so that
// every piece of a row that a workgroup reads or writes is at least 128 bytes long (with 64 x 64 tiles and 64-byte
// pieces the kernel reached 3.5 TB/s at V = 131072).
constexpr int QW_TILE = 128;
template <typename T>
__global__ __launch_bounds__(256) void quantize_w_kernel(const T* __restrict__ w, int64_t ld, int64_t d, int64_t V,
                                                        uint8_t* __restrict__ wq, uint8_t* __restrict__ wqt,
                                                        int64_t dp, int64_t ldx, int64_t kbv, float inv_scale,
                                                        const float* __restrict__ scale_dev) {
  const Scaler scale = make_scaler<T>(inv_scale, scale_dev);
  __shared__ uint8_t tile[QW_TILE][QW_TILE + 4];
  const int t = threadIdx.x;
  const int64_t j0 = (int64_t)blockIdx.y * QW_TILE, v0 = (int64_t)blockIdx.x * QW_TILE;
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int r = (t >> 3) + 32 * pass, c = (t & 7) * 16;
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
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int vr = (t >> 3) + 32 * pass, jc = (t & 7) * 16;
      uint32_t out[4];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        out[m] = (uint32_t)tile[jc + 4 * m][vr] | ((uint32_t)tile[jc + 4 * m + 1][vr] << 8) |
                 ((uint32_t)tile[jc + 4 * m + 2][vr] << 16) | ((uint32_t)tile[jc + 4 * m + 3][vr] << 24);
      }
      *reinterpret_cast<v4i*>(wqt + (v0 + vr) * ldx + j0 + jc) = (v4i){(int)out[0], (int)out[1], (int)out[2], (int)out[3]};
    }
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

}  // namespace sce
