/*
 * slowrun_ce.h - C ABI of libslowrun_ce.so: fused fp8 LM-head + tanh-softcap +
 * cross-entropy, forward and backward, for AMD MI355X (gfx950).
 *
 * The reference has no FFI for this path: its "binding" is a CUDA source string
 * compiled at import time (tiny/cuda_kernels.py:305-312) and wrapped as the
 * custom op nanogpt::ce_fwd_bwd (tiny/cuda_kernels.py:314-334), called from
 * FusedSoftcappedCrossEntropy.forward/backward (tiny/cuda_kernels.py:336-414).
 * The entry points below are what a binding for that autograd Function needs:
 * plain pointers and sizes, no framework types.
 *
 * Conventions
 *  - every pointer is a device pointer on `device`; the caller owns all memory,
 *    including the saved state and the workspaces; the library allocates no
 *    device memory and keeps no pointer after a call returns;
 *  - all work is enqueued on `stream` (a hipStream_t, NULL = default stream);
 *    no call synchronises with the host;
 *  - return value 0 = success, otherwise an SCE_E* code; sce_last_error() gives
 *    a message for the calling thread;
 *  - X is (N, d) row-major, W is (d, V) row-major (the layout of the reference's
 *    CastedLinearT, tiny/train.py:489-497), targets are int64 with
 *    `ignore_index` marking rows that take no part (tiny/train.py:743).
 */
#ifndef SLOWRUN_CE_H
#define SLOWRUN_CE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SCE_VERSION 4

enum { SCE_F32 = 0, SCE_BF16 = 1 };               /* element types of X, W, dX, dW          */
enum { SCE_REDUCE_NONE = 0, SCE_REDUCE_MEAN = 1 }; /* F.cross_entropy(reduction=...)         */

enum {
  SCE_OK = 0,
  SCE_EINVAL = 1,      /* bad shape, dtype, alignment, null pointer, workspace too small     */
  SCE_EARCH = 2,       /* device is not gfx950                                               */
  SCE_EHIP = 3         /* a HIP runtime call failed                                          */
};

typedef struct sce_shape {
  int64_t N;           /* rows (tokens)                         */
  int64_t d;           /* hidden size, multiple of 16, < 2^22   */
  int64_t V;           /* vocabulary (columns of W), at most 524288; N < 2^24 */
  int32_t n_predict;   /* number of MTP offsets, 1..4           */
  int32_t reserved;
} sce_shape;

typedef struct sce_sizes {
  size_t saved_bytes;        /* state written by sce_forward and read by sce_backward        */
  size_t saved_x_bytes;      /* the same when the quantised W lives in a weight cache        */
  size_t wcache_bytes;       /* size of that weight cache                                    */
  size_t fwd_workspace_bytes;
  size_t bwd_workspace_min_bytes;   /* backward with the smallest row panel (256 rows)       */
  size_t bwd_workspace_bytes;       /* backward with the default row panel (with room for the partial tiles of a
                                       K-split last round of dW where there is to be one; less is accepted)   */
  int64_t bwd_panel_rows;           /* the default row panel                                 */
  /* with sce_args.dlogits_from_forward: */
  size_t dlogits_bytes;             /* `saved` grows by this much (N x V bytes and a little)  */
  size_t bwd_workspace_kept_bytes;  /* and backward needs this workspace, no more             */
  size_t saved_bf16_bytes;          /* `saved` of a forward with operand_dtype = SCE_BF16     */
} sce_sizes;

typedef struct sce_args {
  uint32_t struct_size;      /* sizeof(sce_args), checked                                    */
  int32_t device;            /* HIP device ordinal the pointers live on                      */
  void* stream;              /* hipStream_t                                                  */
  sce_shape shape;

  /* ---- inputs (forward) ---- */
  const void* x;  int32_t x_dtype;  int32_t pad0;  int64_t x_ld;   /* (N,d), row stride in elements */
  const void* w;  int32_t w_dtype;  int32_t pad1;  int64_t w_ld;   /* (d,V), row stride in elements */
  const int64_t* targets;    /* (N,)                                                         */
  const float* mtp_weights;  /* (n_predict,) on the device, or NULL for a single weight 1    */
  double x_s, w_s;           /* fp8 scales: X_q = e4m3(X / x_s), W_q = e4m3(W / w_s).  Doubles, as the Python
                                floats of the reference's call are (tiny/train.py:188-189): the quantiser
                                multiplies by (float)(1.0 / x_s), the dequantiser by (float)x_s, which is
                                what torch's GPU kernels make of x.div(x_s) and of the scales of
                                _scaled_mm (tiny/cuda_kernels.py:340-350)                                   */
  float cap;                 /* z = cap * tanh(u / cap), 0 < cap <= 40                       */
  float grad_scale;          /* multiplies every gradient (tiny/cuda_kernels.py:265)         */
  int64_t ignore_index;
  int32_t reduction;         /* SCE_REDUCE_*                                                 */
  int32_t pad2;

  /* ---- outputs (forward) ---- */
  float* loss;               /* [1] mean over valid rows (written when reduction = mean)     */
  float* losses;             /* (N,) per-row loss, 0 at ignored rows; may be NULL for mean   */
  float* lse;                /* (N,) log-sum-exp of the capped logits; optional              */
  int32_t* argmax;           /* (N,) argmax over V of the uncapped logits; optional          */
  int32_t* n_valid;          /* [2]: number of valid rows, number of out-of-range targets    */

  /* ---- state and scratch ---- */
  void* saved;      size_t saved_bytes;
  void* workspace;  size_t workspace_bytes;

  /* ---- backward ---- */
  const float* grad_output;  /* [1] for reduction = mean, (N,) for reduction = none          */
  void* dx;  int32_t dx_dtype;  int32_t pad3;  int64_t dx_ld;      /* (N,d)                  */
  void* dw;  int32_t dw_dtype;  int32_t pad4;  int64_t dw_ld;      /* (d,V)                  */
  int64_t panel_rows;        /* 0 = as many rows per panel as the workspace allows           */

  /* ---- optional ---- */
  int64_t vocab_limit;       /* columns >= vocab_limit take no part in the softmax (the eager head
                                slices the padded vocabulary, tiny/train.py:741); 0 = all V       */
  void* wcache;              /* NULL, or wcache_bytes of device memory holding the quantised W:
                                forward fills it unless wcache_valid, backward reads it          */
  size_t wcache_bytes;
  int32_t wcache_valid;      /* non-zero: wcache already holds e4m3(W / w_s) of this very W      */
  int32_t norm;              /* non-zero: x is the hidden state h before the trunk's last operation,
                                x = F.rms_norm(h, (d,), eps = norm_eps) (tiny/train.py:397-398,734): forward
                                normalises inside the quantiser, backward needs x again and returns the
                                gradient with respect to h in dx                                  */
  float norm_eps;
  int32_t dlogits_from_forward;  /* 0: backward computes the logit tiles again (nothing N x V is kept between the two
                                calls); non-zero: forward also leaves the dlogits, 8 bits each, at the end of `saved`
                                (saved_bytes or saved_x_bytes, plus dlogits_bytes) and backward is two GEMMs instead of
                                three.  Same value in both calls.  The reference keeps bf16 logits and e5m2 dlogits
                                (tiny/cuda_kernels.py:359-371)                                                       */
  const float* x_s_dev;      /* NULL, or a device float that holds the scale of X: read when the kernels run, not when the
                                call is made, so it may be the result of earlier work on the stream (an amax pass, see
                                sce_amax_scale) and may change between replays of a captured graph; x_s is then ignored.
                                The quantiser then divides (x / s) as torch does for a tensor divisor.  Same in forward
                                and backward (backward reads the value forward used from `saved`)                       */
  const float* w_s_dev;      /* the same for W                                                                           */
  int32_t operand_dtype;     /* 0: X and W go into the GEMM as e4m3 (the training path); SCE_BF16: as bf16, the logits
                                rounded to bf16 before the softcap -- the arithmetic of the eager head under bf16
                                autocast (tiny/train.py:741-743 with CastedLinearT :496-497), for validation losses that
                                compare with the reference's.  Forward only (sce_backward refuses it); x_s, w_s are not
                                used; `saved` is then plain scratch of saved_bf16_bytes                              */
  int32_t pad6;
} sce_args;

/* Library / ABI version (SCE_VERSION of the build). */
int sce_version(void);

/* Message for the last non-zero return code on this thread ("" if none). */
const char* sce_last_error(void);

/* Buffer sizes for a problem shape.  Replaces the torch.empty calls in
 * FusedSoftcappedCrossEntropy.forward/backward (tiny/cuda_kernels.py:359-366,398-401). */
int sce_sizes_for(const sce_shape* shape, sce_sizes* out);

/* Per-tensor scaled cast to OCP e4m3: dst[i] = e4m3_rne(src[i] * (float)(1.0 / scale)), NaN code
 * above 464 like Tensor.to(float8_e4m3fn).  The reciprocal is taken once, in double, rounded to
 * fp32 and multiplied in: this is how torch's GPU kernels divide a tensor by a host scalar (its
 * CPU kernels divide element by element; the results differ in the last bit now and then, and
 * that can move an fp8 tie); bf16 input is scaled in fp32 and rounded to bf16 first, as torch
 * does.  sce_forward quantises X and W the same way.  Replaces
 * x.div(x_s).to(torch.float8_e4m3fn) (tiny/cuda_kernels.py:340-341), which runs on the GPU. */
int sce_quantize_e4m3(const void* src, int32_t src_dtype, void* dst, double scale, size_t n,
                      int32_t device, void* stream);

/* The same with the scale in device memory (a 0-dim tensor): dst[i] = e4m3_rne(src[i] / *scale_dev), a true
 * division, which is what torch computes for a tensor divisor; nothing is read on the host. */
int sce_quantize_e4m3_dev(const void* src, int32_t src_dtype, void* dst, const float* scale_dev, size_t n,
                          int32_t device, void* stream);

/* *scale_out (a device float) = max |src[i]| / 448, the per-tensor "amax" scale of the fp8 cast, for
 * x_s_dev / w_s_dev; NaN if any element is NaN.  Replaces a host-side `float(t.abs().max()) / 448` (the reference's
 * scales are constants, tiny/train.py:188-189; a trainer that rescales per step does this). */
int sce_amax_scale(const void* src, int32_t src_dtype, size_t n, float* scale_out, int32_t device, void* stream);

/* dst (cols, rows) = transpose of src (rows, cols), one byte per element.  Replaces
 * transpose_copy (tiny/cuda_kernels.py:56-78) for callers that still want it; the fused
 * path itself never materialises a transposed N x V matrix. */
int sce_transpose_bytes(const void* src, void* dst, int64_t rows, int64_t cols,
                        int32_t device, void* stream);

/* Forward: quantise X and W, contract on fp8 MFMA, softcap, online log-sum-exp, loss.
 * Replaces FusedSoftcappedCrossEntropy.forward (tiny/cuda_kernels.py:336-373) and the
 * kernel it launches (tiny/cuda_kernels.py:125-240).  Uses args->workspace
 * (fwd_workspace_bytes) and fills args->saved. */
int sce_forward(const sce_args* args);

/* sce_forward without a workspace: the scratch that sce_forward takes from args->workspace (the partial row
 * statistics of the vocabulary splits) lives in a static device array of the library, 8 MiB on every GPU the
 * library has run on, until the process ends.  No counterpart in the reference; it is for callers that cannot
 * allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The call allocates
 * nothing and frees nothing; args->workspace and args->workspace_bytes are ignored, every other field means what it
 * means to sce_forward, and the results are the same bits.  Limit: ceil(N / 256) * 256 * S <= 524288, S the number of
 * vocabulary splits (8 to 16; 8 at N = 65536, V = 50304), else SCE_EINVAL with a message.  All calls on one device
 * share the one array: calls that overlap in time on the same device (two streams, two threads) race. */
int sce_forward_noalloc(const sce_args* args);

/* Backward: dX = dlogits * W_q^T, dW = X_q^T * dlogits on the MFMA, the dlogits either as the forward pass left them
 * (dlogits_from_forward) or formed again from recomputed logit tiles, row panel by row panel.  Replaces
 * FusedSoftcappedCrossEntropy.backward (tiny/cuda_kernels.py:375-414) and the dlogits half
 * of the reference kernel (tiny/cuda_kernels.py:242-301).  Needs the `saved` buffer of the
 * matching sce_forward call, the same shape/scales/cap/targets, and a workspace of
 * bwd_workspace_kept_bytes (dlogits_from_forward) or at least bwd_workspace_min_bytes. */
int sce_backward(const sce_args* args);

/* ---- optional per-kernel timing (off by default) --------------------------------------
 * No counterpart in the reference (it times whole steps with torch.cuda.synchronize,
 * tiny/train.py:1408-1452).  While enabled, sce_forward / sce_backward record a HIP event
 * pair on the caller's stream around each group of launches; sce_timing_read waits for the
 * recorded events and returns the accumulated time and number of groups per kind. */
enum {
  SCE_K_QUANT = 0,       /* X and W quantisation                                             */
  SCE_K_FWD = 1,         /* fused logits + softcap + online LSE (one launch per forward)     */
  SCE_K_FWD_REDUCE = 2,  /* combine of the V-splits and the mean                             */
  SCE_K_BWD_PREP = 3,    /* row scales, scaled X^T, rows grouped by target                   */
  SCE_K_RECOMPUTE = 4,   /* logit recompute -> dlogits panel in the workspace (one launch per panel) */
  SCE_K_DX = 5,          /* dX panel GEMM                                                    */
  SCE_K_DW = 6,          /* dW panel GEMM                                                    */
  SCE_K_DW_FINAL = 7,    /* one-hot part of dW, scaling, cast                                */
  SCE_K_COUNT = 8
};
typedef struct sce_timing {
  double ms[SCE_K_COUNT];
  int64_t launches[SCE_K_COUNT];
} sce_timing;
int sce_timing_enable(int on);            /* also clears the accumulators */
int sce_timing_read(sce_timing* out);

/* ---- measurement aids (no counterpart in the reference) ---------------------------------
 * What the matrix pipe and the MFMA main loop of this library reach on their own, for the ceiling figures that
 * `python -m slowrun_amd.ceiling` reports.  Both synchronise with the host (they time `reps` launches with HIP events)
 * and return the rate in TFLOP/s and the shader clock that the kernels themselves saw (their cycle counter against the
 * 100 MHz reference counter; median over workgroups).  scratch: device memory, 1 KiB per 256 x 256 tile and 16 KiB more.
 *  sce_bench_mfma: 16 independent v_mfma_f32_32x32x64_f8f6f4 per wave and round, operands in registers, no memory traffic;
 *                  random_bytes: NULL (all operands 1.0) or random_bytes_size >= 64 KiB x (4 x CUs) device bytes that become
 *                  the operands (a smaller buffer is refused).
 *  sce_bench_gemm: C = A B^T through the library's main loop (256 x 256 tiles, global -> LDS -> MFMA), the sums of the
 *                  accumulators stored; A is (M, K) and B (N, K) e4m3 bytes with a row stride of K + 128 bytes. */
int sce_bench_mfma(const void* random_bytes, size_t random_bytes_size, int32_t iters, int32_t reps, void* scratch, size_t scratch_bytes,
                   int32_t device, void* stream, double* tflops, double* shader_mhz);
int sce_bench_gemm(const void* A, const void* B, int64_t M, int64_t N, int64_t K, int32_t reps, void* scratch, size_t scratch_bytes,
                   int32_t device, void* stream, double* tflops, double* shader_mhz);
/*  sce_bench_floor: the main loops of the three big kernels alone -- the tile walk of the forward kernel (which = SCE_K_FWD),
 *                  all dX panels (SCE_K_DX), the dW launch (SCE_K_DW) -- in their own operand layouts, tile orders and MFMA
 *                  variants, with nothing for an epilogue (a checksum per thread).  args: as passed to a forward call with
 *                  dlogits_from_forward and to the matching backward call, after both have run (saved: X_q, W_q and the
 *                  dlogits; workspace: the scaled transposed X); all-zero buffers of those sizes give the time of the same
 *                  instruction stream on operands that draw little power.  N at most 131072.  Returns the time of one pass in
 *                  ms and the shader clock the kernels saw.  scratch as for sce_bench_gemm, 1 KiB per workgroup of the largest grid. */
int sce_bench_floor(const sce_args* args, int32_t which, int32_t reps, void* scratch, size_t scratch_bytes, double* ms_per_pass,
                    double* shader_mhz);

/* ---- test aid (no counterpart in the reference) --------------------------------------------
 * A forward pass with dlogits_from_forward computes its target logits ahead of the forward kernel, from a tile of gathered
 * rows of the quantised W, while W_q^T is smaller than 4 GiB (the reach of that tile's 32-bit offsets), and inside the
 * forward kernel, out of its accumulators, beyond.  This sets the size in bytes from which the second way is taken
 * (0 or less: back to 4 GiB), so that a test can run it at a size it can afford.  Process-wide; returns the previous
 * value.  The results of the two ways are the same bit for bit in the losses and within the tolerances in the
 * gradients (the target entries of a block take part in nothing either way). */
int64_t sce_test_set_gather_limit(int64_t bytes);

#ifdef __cplusplus
}
#endif
#endif
