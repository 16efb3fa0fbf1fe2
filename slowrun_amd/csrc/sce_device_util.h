// Small device helpers of the loss-head kernels: fast transcendentals, e4m3 and bf16 conversions, scales that
// may live on the device, the XCD-aware tile orders (internal header).
// Part of the one translation unit sce_kernels.hip, which includes it after the headers it builds on.
#pragma once

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
// the same value through the hardware conversion (v_cvt_pk_bf16_f32: round to nearest even; a NaN stays a NaN, with
// whatever payload the hardware gives it)
__device__ __forceinline__ float round_to_bf16_hw(float f) { return (float)(__bf16)f; }

// two floats -> two e4m3 bytes (low half of the result).  v_cvt_pk_fp8_f32 on gfx950 is OCP
// e4m3fn, round to nearest even, 464 -> 448 and anything larger -> NaN code: the same rule as
// Tensor.to(torch.float8_e4m3fn).
__device__ __forceinline__ uint32_t cvt2_e4m3(float a, float b) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}
__device__ __forceinline__ uint32_t cvt4_e4m3(float a, float b, float c, float d) {
  // (the instruction keeps the other half of its destination: both halves are written here, so what the destination held
  // does not matter, and `a` as that old value lets the compiler convert in place instead of clearing a register first)
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, __float_as_int(a), false);
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

// a pointer that is the same in every lane, moved to scalar registers
__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* q) {
  const uint64_t u = (uint64_t)(uintptr_t)q;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)u), hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(u >> 32));
  return (const uint8_t*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

}  // namespace sce
