/* hpfp8 -- C ABI of the MI355X (gfx950) FP8 mixed-precision linear path.
 *
 * Every entry point takes raw DEVICE pointers, sizes and a HIP stream, enqueues its kernels on
 * that stream and returns without synchronizing.  Return value: HPFP8_OK (0) or a negative
 * HPFP8_ERR_* code; hpfp8_last_error() then gives a human-readable message for the calling
 * thread.  No exception crosses this boundary and no entry point allocates device memory.
 *
 * Data conventions
 *   bf16 tensors   : uint16 bit patterns, row-major, 16-byte aligned base
 *   E4M3 codes     : uint8 (OCP E4M3FN: bias 7, max 448, NaN = S.1111.111, no Inf)
 *   scale          : fp32, quantize multiplier   448 / max(amax, 1e-12)
 *   scale_inv      : fp32, dequantize multiplier max(amax, 1e-12) / 448   (what the GEMMs consume)
 *   code           : e4m3_rne(clamp(float(x) * scale, -448, 448))
 *   non-finite x   : IEEE rules with amax and clamp keeping NaN: a NaN in a scaling group makes the group's
 *                    scale, scale_inv and codes NaN; +-Inf gives scale 0, scale_inv Inf, codes +-0 for the
 *                    finite elements and NaN for the infinite ones.  Dequantized values and GEMM outputs fed
 *                    by such a group are NaN.  The sign bit of a NaN code is unspecified.
 *
 * What each entry point stands in for.  The reference (mindspore-ai/hyper-parallel) has no FP8
 * kernels and no C/FFI boundary on its torch platform: a linear there is aten::linear called at
 * hyper_parallel/core/shard/_op_dispatch.py:277-283 with the operand roles checked in
 * hyper_parallel/core/shard/ops/parallel_matmul.py:344-404 (weight [out, in], contraction over
 * the last dim of both), its backward is torch autograd of that op, and the gradient bucket
 * cast sites are hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108 (cast in) and :116-135
 * (cast back, then * grad_scale).  Each declaration below names the site it replaces.
 */
#ifndef HPFP8_H_
#define HPFP8_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* hpfp8_stream_t; /* a hipStream_t; NULL is the default stream */

enum {
  HPFP8_OK = 0,
  HPFP8_ERR_ARG = -1,    /* null pointer / bad flag */
  HPFP8_ERR_SHAPE = -2,  /* shape not supported (not a multiple of 128, too large, negative) */
  HPFP8_ERR_ALIGN = -3,  /* pointer not 16-byte aligned */
  HPFP8_ERR_LAUNCH = -4, /* HIP reported a launch error */
  HPFP8_ERR_DEVICE = -5  /* not a gfx950 device */
};

/* Output element type of the GEMMs. */
enum { HPFP8_OUT_BF16 = 0, HPFP8_OUT_F32 = 1 };

/* Library version (major*10000 + minor*100 + patch). */
int hpfp8_version(void);
/* Message of the last failing call made by this thread ("" if none). */
const char* hpfp8_last_error(void);
/* HPFP8_OK if the current HIP device is gfx950. */
int hpfp8_check_device(void);

/* ---- amax and per-tensor cast ----------------------------------------------------------------
 * Stand in for the dtype cast hooks of the torch platform, TorchPlatform.cast_fp_tensor
 * (hyper_parallel/platform/torch/platform.py:587-597), for the FP8 target type that hook cannot
 * express (a cast plus a scale). */

/* amax_out[0] = max |x[i]| as fp32 over n bf16 values (0 for n == 0). */
int hpfp8_amax_bf16(const void* x, int64_t n, float* amax_out, hpfp8_stream_t stream);

/* q[i] = code(x[i]) with the scale derived on the device from amax[0]; scale / scale_inv
 * (each may be NULL) receive the two multipliers. */
int hpfp8_cast_per_tensor_bf16(const void* x, int64_t n, const float* amax, void* q, float* scale,
                               float* scale_inv, hpfp8_stream_t stream);

/* amax followed by cast: amax (fp32[1], required) is written then consumed.  Up to 4 Mi elements, and when
 * scale_inv is asked for, this is one pass over x (3 bytes per element): the grid keeps x in registers and agrees
 * on the maximum through the amax word, using the scale_inv word as its arrival count until the value is stored
 * there; larger tensors take the two passes above.  Either way amax holds max |x| as a clean fp32 and scale_inv
 * its value when the call's kernels have finished. */
int hpfp8_quantize_per_tensor_bf16(const void* x, int64_t n, void* q, float* amax, float* scale,
                                   float* scale_inv, hpfp8_stream_t stream);

/* The same in ONE launch, for tensors of up to 4 Mi elements (more is HPFP8_ERR_SHAPE): `sync` points at 512 bytes of
 * device memory (256-byte aligned) that the caller keeps for this purpose, zero before the first call; every call
 * finds it zero and leaves it zero (the last workgroup to finish with it clears it), so calls that follow each other
 * on a stream -- or replays of a captured graph -- need nothing cleared in between.  Calls that may overlap on the
 * GPU need a `sync` of their own each.  amax, scale and scale_inv (each may be NULL) receive max |x| and the two
 * multipliers.  Same codes and scales as hpfp8_quantize_per_tensor_bf16. */
int hpfp8_quantize_per_tensor_sync_bf16(const void* x, int64_t n, void* q, float* amax, float* scale, float* scale_inv,
                                        uint32_t* sync, hpfp8_stream_t stream);

/* hpfp8_quantize_per_tensor_bf16 for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the amax word is not supplied by the caller but lives in
 * 256 bytes of device memory the library holds on every GPU it runs on until the process ends, so the call
 * needs no workspace and allocates nothing.  No counterpart in the reference.  Same codes, scale and scale_inv
 * as hpfp8_quantize_per_tensor_bf16.  At most 4,194,304 elements (the one-pass form; more is HPFP8_ERR_SHAPE).
 * All calls on one GPU share that memory: calls that overlap on one GPU (different streams without ordering)
 * race and may produce wrong scales; calls ordered on a stream, or separated by events, are safe.  The
 * memory's address is resolved on the first call per device, or by hpfp8_check_device() made with that device
 * current (do one of the two before capturing a graph). */
int hpfp8_quantize_per_tensor_noalloc_bf16(const void* x, int64_t n, void* q, float* scale, float* scale_inv,
                                           hpfp8_stream_t stream);

/* Measurement aid, not part of the path: the memory traffic of hpfp8_quantize_128x1_t_kmajor_bf16 (q == NULL) or of
 * hpfp8_quantize_1x128_and_128x1_t_bf16 (q != NULL) and nothing else -- the same tile loads, in the same tile order,
 * and stores of the same sizes at the same addresses, whose contents are meaningless.  bench.py times it beside the
 * real kernels: what it reaches is what the access pattern allows on the machine. */
int hpfp8_debug_transpose_traffic_model(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t, void* q,
                                        hpfp8_stream_t stream);

/* Test hook, not part of the path: how many times a workgroup of the one-pass per-tensor quantizer polls for the
 * rest of its grid before it computes the tensor's maximum alone (default 256 polls, a few hundred microseconds
 * at most; a resident grid needs a handful).  0 forces that path, which must give the same results.  The value is
 * process-wide and stored atomically: it may be set from any thread and takes effect with the next launch. */
void hpfp8_debug_set_spin_limit(uint32_t polls);

/* ---- blockwise quantizers --------------------------------------------------------------------
 * Operand preparation for the linear of hyper_parallel/core/shard/_op_dispatch.py:277-283. */

/* Activations / gradient buckets: x[rows, cols] bf16, one scale per 128 contiguous values.
 * q[rows, cols]; scale (may be NULL) and scale_inv are [rows, cols/128]. */
int hpfp8_quantize_1x128_bf16(const void* x, int64_t rows, int64_t cols, void* q, float* scale,
                              float* scale_inv, hpfp8_stream_t stream);

/* Same codes; scale / scale_inv written k-block-major, [cols/128, rows]: element (row, g) at
 * [g * rows + row].  This is the layout the GEMMs read with unit stride over a fragment's rows
 * (pass sa_stride_m = 1, sa_stride_k = rows). */
int hpfp8_quantize_1x128_kmajor_bf16(const void* x, int64_t rows, int64_t cols, void* q, float* scale,
                                     float* scale_inv, hpfp8_stream_t stream);

/* Weights: w[rows, cols] bf16, one scale per 128x128 block.  q[rows, cols]; q_t (may be NULL)
 * receives the transposed codes [cols, rows] that dgrad consumes, with row stride ld_t bytes
 * (>= rows, multiple of 16; a stride that is an odd multiple of 128 avoids HBM channel camping);
 * scale (may be NULL) and scale_inv are [rows/128, cols/128]. */
int hpfp8_quantize_128x128_bf16(const void* w, int64_t rows, int64_t cols, void* q, void* q_t, int64_t ld_t,
                                float* scale, float* scale_inv, hpfp8_stream_t stream);

/* wgrad operands: x[m, k] bf16, one scale per 128 consecutive ROWS of a column, written
 * transposed: q_t[k, m] with row stride ld_t bytes (>= m, multiple of 16); scale_t (may be NULL)
 * and scale_inv_t are [k, m/128]. */
int hpfp8_quantize_128x1_t_bf16(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t, float* scale_t,
                                float* scale_inv_t, hpfp8_stream_t stream);

/* Same codes; scale_t / scale_inv_t written block-major, [m/128, k]: element (col, b) at
 * [b * k + col]. */
int hpfp8_quantize_128x1_t_kmajor_bf16(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t,
                                       float* scale_t, float* scale_inv_t, hpfp8_stream_t stream);

/* Both quantizations of one bf16 matrix from one read of it: the 1x128 form (forward / dgrad
 * operand: q[m, k], scales [m, k/128], or [k/128, m] when kmajor != 0) and the transposed 128x1 form
 * (wgrad operand: q_t[k, m] with row stride ld_t, scales [k, m/128], or [m/128, k] when kmajor != 0).
 * Codes and scales are bit-identical to hpfp8_quantize_1x128[_kmajor]_bf16 and
 * hpfp8_quantize_128x1_t[_kmajor]_bf16 on the same input.  m and k multiples of 128.  Serves the same
 * call site as those two (operand preparation for hyper_parallel/core/shard/_op_dispatch.py:277-283,
 * forward and backward). */
int hpfp8_quantize_1x128_and_128x1_t_bf16(const void* x, int64_t m, int64_t k, int kmajor, void* q, float* scale,
                                          float* scale_inv, void* q_t, int64_t ld_t, float* scale_t,
                                          float* scale_inv_t, hpfp8_stream_t stream);

/* Bias gradient.  The backward of the linear the reference dispatches (aten::linear at
 * hyper_parallel/core/shard/_op_dispatch.py:277-283, differentiated by torch autograd) sums grad_out over the tokens
 * for the bias.  Here that sum comes out of the pass that already reads every element of grad_out:
 *   hpfp8_quantize_128x1_t_colsum_bf16  hpfp8_quantize_1x128_and_128x1_t_bf16 with kmajor = 1 (or, with q == NULL,
 *                                       hpfp8_quantize_128x1_t_kmajor_bf16; pow2 != 0: the _pow2 forms), which also
 *                                       writes colsum_partial[m/128, k] (fp32): per 128-row block and column the sum of
 *                                       the block's rows;
 *   hpfp8_column_sum_finish             out[col] = the partial sums of a column added in block order onto +0, as fp32
 *                                       (out_f32) and / or rounded once to bf16 (out_bf16); either may be NULL;
 *   hpfp8_column_sum_bf16               both steps for a matrix that is not being quantized (x[m, k], row stride ld
 *                                       elements, any m, k a multiple of 128; partial[ceil(m/128), k] is caller-owned
 *                                       scratch), with the same bits as the fused form.
 * The additions inside a block run in a fixed order (stated with tile_column_sums in csrc/quantize.hip and restated
 * by the CPU oracle), so the result is reproducible bit for bit. */
int hpfp8_quantize_128x1_t_colsum_bf16(const void* x, int64_t m, int64_t k, void* q, float* scale, float* scale_inv, void* q_t,
                                       int64_t ld_t, float* scale_t, float* scale_inv_t, int pow2, float* colsum_partial,
                                       hpfp8_stream_t stream);
int hpfp8_column_sum_finish(const float* partial, int64_t blocks, int64_t cols, void* out_bf16, float* out_f32,
                            hpfp8_stream_t stream);
int hpfp8_column_sum_bf16(const void* x, int64_t m, int64_t k, int64_t ld, float* partial, void* out_bf16, float* out_f32,
                          hpfp8_stream_t stream);

/* Power-of-two scales (an optional recipe; the stated one keeps plain fp32 scales): scale_inv is
 * amax_c / 448 rounded up to the next power of two and scale its exact reciprocal, everything else as in
 * the entry point of the same name without _pow2.  Such a scale_inv's fp32 exponent field is its E8M0
 * code, which gfx950's block-scaled matrix instruction applies by itself: hpfp8_gemm_blockwise_pow2
 * below.  No counterpart in the reference; same call sites as the plain forms. */
int hpfp8_quantize_1x128_kmajor_pow2_bf16(const void* x, int64_t rows, int64_t cols, void* q, float* scale,
                                          float* scale_inv, hpfp8_stream_t stream);
int hpfp8_quantize_128x128_pow2_bf16(const void* w, int64_t rows, int64_t cols, void* q, void* q_t, int64_t ld_t,
                                     float* scale, float* scale_inv, hpfp8_stream_t stream);
int hpfp8_quantize_128x1_t_kmajor_pow2_bf16(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t,
                                            float* scale_t, float* scale_inv_t, hpfp8_stream_t stream);
int hpfp8_quantize_1x128_and_128x1_t_pow2_bf16(const void* x, int64_t m, int64_t k, int kmajor, void* q, float* scale,
                                               float* scale_inv, void* q_t, int64_t ld_t, float* scale_t,
                                               float* scale_inv_t, hpfp8_stream_t stream);
int hpfp8_swiglu_quantize_1x128_pow2_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int kmajor, void* q,
                                          float* scale, float* scale_inv, void* act, hpfp8_stream_t stream);

/* SwiGLU fused with the 1x128 quantization of its result, the activations of the down projection
 * (the step after the gate/up linear of a DeepSeekV3 MLP; in the reference this is eager
 * F.silu(gate) * up between two aten::linear calls dispatched at
 * hyper_parallel/core/shard/_op_dispatch.py:277-283).  h[rows, 2 * inter] bf16 with row stride ld_h
 * elements: gate = columns [0, inter), up = columns [inter, 2 * inter).
 *   act = bf16( bf16(silu(gate)) * up ),  silu(g) = g / (1 + exp(-g)) in fp32 with the exponential
 *   defined operation by operation in csrc/quantize.hip (exp_spec) and restated in the oracle,
 * quantized like hpfp8_quantize_1x128[_kmajor]_bf16: q[rows, inter], scales [rows, inter/128] or
 * (kmajor != 0) [inter/128, rows].  act (bf16 [rows, inter]) is also written when not NULL. */
int hpfp8_swiglu_quantize_1x128_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int kmajor, void* q,
                                     float* scale, float* scale_inv, void* act, hpfp8_stream_t stream);
/* The same with silu from the hardware's base-2 exponential and reciprocal approximations (each within
 * one unit in the last place of fp32) instead of the exactly specified sequence: the kernel is then bound by
 * memory, not arithmetic (about twice as fast).  the bf16 silu can differ from the exact form's by one unit in the last
 * place (act, its product with up, by two) in about one element per ten thousand, as two GPU implementations of the eager graph differ from each
 * other; q, scale and scale_inv are the exact 1x128 quantization of the act this call writes.  pow2 (0 / 1)
 * selects power-of-two scales as in hpfp8_swiglu_quantize_1x128_pow2_bf16. */
int hpfp8_swiglu_quantize_1x128_fast_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int kmajor, int pow2,
                                          void* q, float* scale, float* scale_inv, void* act, hpfp8_stream_t stream);

/* SwiGLU fused with both quantized forms of its result (training: the down projection's forward operand and
 * its wgrad operand from one read of the gate/up output; the bf16 activation is never written): the results of
 * hpfp8_swiglu_quantize_1x128_bf16 (fast == 0) or _fast_bf16 (fast != 0) with k-block-major scales
 * (q[rows, inter], scale / scale_inv [inter/128, rows]) and of hpfp8_quantize_128x1_t_kmajor_bf16 applied to that
 * activation (q_t[inter, rows] with row stride ld_t, scale_t / scale_inv_t [rows/128, inter]), bit for bit.
 * rows and inter multiples of 128. */
int hpfp8_swiglu_quantize_1x128_and_128x1_t_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int fast,
                                                 void* q, float* scale, float* scale_inv, void* q_t, int64_t ld_t,
                                                 float* scale_t, float* scale_inv_t, hpfp8_stream_t stream);

/* Backward of act = silu(gate) * up (the autograd of the same eager graph): h[rows, 2 * inter] = gate | up as in the
 * forward call, dact[rows, inter] the gradient of act (contiguous), dh[rows, 2 * inter] (row stride ld_dh) receives
 * d gate | d up, all bf16:  d up = dact * bf16(silu(gate)),  d gate = dact * up * (sig + silu * (1 - sig)) with
 * sig = 1 / (1 + exp(-gate)) from the hardware's exponential and reciprocal, in fp32, one rounding each.
 * inter a multiple of 8. */
int hpfp8_swiglu_backward_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, const void* dact, void* dh,
                               int64_t ld_dh, hpfp8_stream_t stream);

/* hpfp8_swiglu_backward_bf16 fused with both quantized forms of its result (training: the output gradient of the
 * gate/up projection as its dgrad operand and its wgrad operand, from one read of h and dact; the bf16 gradient
 * d gate | d up is never written): with dh the [rows, 2 * inter] tensor hpfp8_swiglu_backward_bf16 would write,
 * q[rows, 2 * inter], scale / scale_inv [2 * inter / 128, rows] are hpfp8_quantize_1x128_kmajor_bf16(dh) and
 * q_t[2 * inter, rows] (row stride ld_t), scale_t / scale_inv_t [rows / 128, 2 * inter] are
 * hpfp8_quantize_128x1_t_kmajor_bf16(dh), bit for bit.  rows and inter multiples of 128; dact contiguous. */
int hpfp8_swiglu_backward_quantize_1x128_and_128x1_t_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h,
                                                          const void* dact, void* q, float* scale, float* scale_inv,
                                                          void* q_t, int64_t ld_t, float* scale_t, float* scale_inv_t,
                                                          hpfp8_stream_t stream);

/* Byte transpose of a code matrix: q[rows, cols] (row stride ld) -> q_t[cols, rows] (row stride ld_t);
 * rows, cols multiples of 128.  128x128 scaling blocks are symmetric, so this turns the codes of a
 * weight into its dgrad operand without requantizing, e.g. after FP8 shards were all-gathered: the
 * float8 all-gather extension point the reference leaves as a stub
 * (hyper_parallel/platform/torch/fully_shard/param.py:299-310). */
int hpfp8_transpose_codes(const void* q, int64_t rows, int64_t cols, int64_t ld, void* q_t, int64_t ld_t,
                          hpfp8_stream_t stream);

/* ---- dequantizers ----------------------------------------------------------------------------
 * The cast-back site hyper_parallel/core/hsdp/hsdp_grad_buffer.py:116-125: out = bf16(decode(q)
 * * scale_inv); when grad_scale != 1 the bf16 result is multiplied by it and rounded again. */
int hpfp8_dequantize_1x128_bf16(const void* q, const float* scale_inv, int64_t rows, int64_t cols,
                                void* out, float grad_scale, hpfp8_stream_t stream);
/* The cast back of the per-parameter cast hooks, HSDPGradHook._cast_hook
 * (hyper_parallel/core/hsdp/hsdp_grad_hook.py:32-40: `.to(origin_dtype)` after the reduction) and
 * HSDPAsyncGradHook._post_process (hyper_parallel/core/hsdp/hsdp_async_grad_hook.py:23-39), for a tensor that
 * hpfp8_quantize_per_tensor_bf16 cast in: out[i] = decode(q[i]) * scale_inv[0] for n codes, one multiplication
 * in fp32, rounded once to bf16 (HPFP8_OUT_BF16) or left in fp32 (HPFP8_OUT_F32). */
int hpfp8_dequantize_per_tensor(const void* q, int64_t n, const float* scale_inv, void* out, int out_type,
                                hpfp8_stream_t stream);
int hpfp8_dequantize_128x128_bf16(const void* q, const float* scale_inv, int64_t rows, int64_t cols,
                                  void* out, hpfp8_stream_t stream);
/* main_grad[i] += (decode(q[i]) * scale_inv) * grad_scale, all in fp32 (two multiplications, then the
 * addition): a reduced FP8 gradient added onto the fp32 main gradient in one pass, the
 * `main_grad += reduced_grad` of hyper_parallel/platform/torch/fully_shard/param.py:160-167 under
 * MixedPrecisionPolicy.apply_grad_on_fp32_main_grad (platform/torch/fully_shard/utils.py:24). */
int hpfp8_dequantize_1x128_accumulate_f32(const void* q, const float* scale_inv, int64_t rows, int64_t cols,
                                          float* main_grad, float grad_scale, hpfp8_stream_t stream);

/* ---- gradient bucket: pack + quantize, dequantize + unpack -------------------------------------
 * The FP8 form of HSDPGradBuffer._copy_grad_to_unsharded_buffer and ._set_grad_data
 * (hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108, :116-135).  The bucket is `shards` rows of
 * row_elems elements (a multiple of 128); parameter e owns elements [offsets[e], offsets[e] +
 * numels[e]) of every row, offsets ascending multiples of 128 starting at 0, the gap up to the next
 * offset (or the end of the row) is padding.  grads, numels, offsets are HOST arrays of `entries`
 * items; grads[e] is a device pointer to bf16 data.
 *
 * pack:   row s of the bucket = chunk s of every gradient (grads[e] holds shards * numels[e]
 *         elements, chunk s = elements [s * numels[e], (s + 1) * numels[e])), quantized in 1x128
 *         groups along the row: q[shards, row_elems] E4M3, scale / scale_inv [shards, row_elems / 128]
 *         (scale may be NULL).  Padding is written as zero codes.  Same codes and scales as
 *         hpfp8_quantize_1x128_bf16 on the packed bf16 rows.
 * unpack: one (reduced) row q[row_elems], scale_inv[row_elems / 128] -> grads[e][0 .. numels[e]) =
 *         bf16(decode * scale_inv), then, when grad_scale != 1, bf16(that * grad_scale): the order of
 *         hsdp_grad_buffer.py:121-125.  Same values as hpfp8_dequantize_1x128_bf16 on the row. */
int hpfp8_bucket_pack_quantize_bf16(const void* const* grads, const int64_t* numels, const int64_t* offsets,
                                    int entries, int shards, int64_t row_elems, void* q, float* scale,
                                    float* scale_inv, hpfp8_stream_t stream);
int hpfp8_bucket_unpack_dequantize_bf16(void* const* grads, const int64_t* numels, const int64_t* offsets,
                                        int entries, int64_t row_elems, const void* q, const float* scale_inv,
                                        float grad_scale, hpfp8_stream_t stream);

/* ---- scaled FP8 GEMMs -------------------------------------------------------------------------
 * Replace aten::linear (forward) and its autograd backward (dgrad, wgrad) as called from
 * hyper_parallel/core/shard/_op_dispatch.py:277-283.
 *
 *   c[m, n] = sum_kb  sa(m, kb) * sb(n, kb) * ( sum_{k in block kb} a[m, k] * b[n, k] )  (+ bias[n])
 *
 * a[M, K] and b[N, K] are E4M3 codes with K contiguous and row strides lda / ldb bytes (>= K,
 * multiples of 16); K, N multiples of 128; fp32 accumulation, k-blocks ascending; one rounding to
 * bf16 at the end (or fp32 output).
 *   sa(m, kb) = sa[m * sa_stride_m + kb * sa_stride_k]
 *   sb(n, kb) = sb[(n / sb_gran) * sb_stride_n + kb * sb_stride_k],  sb_gran = 128 or 1
 * Uses:  forward  a = x codes (1x128),  b = W codes (128x128),            sb_gran = 128
 *        dgrad    a = grad_out codes,   b = W^T codes, W's scales with swapped strides
 *        wgrad    a = grad_out^T codes (128x1 requant), b = x^T codes,    sb_gran = 1; the b scales must
 *                 then be k-block-major: sb_stride_n = 1, sb_stride_k >= N (what the *_kmajor quantizers write)
 * bias: bf16[N] or NULL.  out_type HPFP8_OUT_BF16 / HPFP8_OUT_F32; ldc = row stride of c in
 * elements, a multiple of 8 (bf16) or 4 (fp32): rows are written in 16-byte pieces.  Scale strides are
 * non-negative; each scale array must span less than 2 GiB and a row stride of a, b or c stay below 8 MiB
 * (HPFP8_ERR_SHAPE otherwise); the code matrices and c themselves may be of any size.  accumulate != 0
 * (fp32 output only) adds onto c instead of overwriting it, the fp32 main-grad bookkeeping of
 * hyper_parallel/platform/torch/fully_shard/param.py:134-167: the old value of an element is the starting
 * value of its sum, the k-blocks are added onto it in ascending order. */
int hpfp8_gemm_blockwise(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                         const void* b, int64_t ldb, const float* sb, int64_t sb_stride_n, int64_t sb_stride_k,
                         int sb_gran, int64_t M, int64_t N, int64_t K, const void* bias, void* c,
                         int64_t ldc, int out_type, int accumulate, hpfp8_stream_t stream);

/* hpfp8_gemm_blockwise for scales that are powers of two (what the _pow2 quantizers write): the matrix
 * instruction applies them as E8M0 block scales and sums the k-blocks itself, so the kernel spends no
 * arithmetic on scaling.  Only the exponent field of a scale is used (mantissa bits are ignored, the
 * sign must be +).  Same arguments and limits as hpfp8_gemm_blockwise.  Results
 * agree with hpfp8_gemm_blockwise on the same operands to fp32 rounding (the order of the fp32
 * additions differs), and are exact on the same integer-valued cases. */
int hpfp8_gemm_blockwise_pow2(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                              const void* b, int64_t ldb, const float* sb, int64_t sb_stride_n, int64_t sb_stride_k,
                              int sb_gran, int64_t M, int64_t N, int64_t K, const void* bias, void* c, int64_t ldc,
                              int out_type, int accumulate, hpfp8_stream_t stream);

/* The gate/up projection of a SwiGLU MLP with the activation and the 1x128 quantization of the down projection's
 * input as the GEMM's epilogue: no bf16 gate/up tensor is written or read (the eager graph this replaces is two
 * aten::linear calls dispatched at hyper_parallel/core/shard/_op_dispatch.py:277-283 with F.silu(gate) * up
 * between them).  a[M, K], sa as in hpfp8_gemm_blockwise; b = codes of W_gate_up [2 * inter, K] (gate rows
 * [0, inter), up rows [inter, 2 * inter); must span less than 2 GiB) with 128x128 scales
 * sb(n / 128, kb) = sb[(n / 128) * sb_stride_n + kb * sb_stride_k]; inter and K multiples of 128.
 *   h = bf16(gate | up) as hpfp8_gemm_blockwise[_pow2] (pow2 = 0 / 1: which of the two, by the operands' scales)
 *       would write it; act = bf16(bf16(silu(gate)) * up) as hpfp8_swiglu_quantize_1x128_bf16 (fast = 0) or
 *       hpfp8_swiglu_quantize_1x128_fast_bf16 (fast = 1) defines it;
 *   q[M, inter] (row stride ldq bytes, a multiple of 16), scale (may be NULL) and scale_inv [inter / 128, M]
 *       (k-block-major): bit for bit what those two calls in a row give, with power-of-two scales when
 *       pow2_out = 1. */
int hpfp8_gemm_blockwise_swiglu_quantize(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m,
                                         int64_t sa_stride_k, const void* b, int64_t ldb, const float* sb,
                                         int64_t sb_stride_n, int64_t sb_stride_k, int64_t M, int64_t inter, int64_t K,
                                         int fast, int pow2, int pow2_out, void* q, int64_t ldq, float* scale,
                                         float* scale_inv, hpfp8_stream_t stream);

/* Per-tensor scales: c = (a . b^T) * (sa_inv[0] * sb_inv[0]) (+ bias), accumulation over the whole
 * K inside the matrix cores.  K a multiple of 128, N a multiple of 128. */
int hpfp8_gemm_per_tensor(const void* a, int64_t lda, const float* sa_inv, const void* b, int64_t ldb,
                          const float* sb_inv, int64_t M, int64_t N, int64_t K, const void* bias, void* c,
                          int64_t ldc, int out_type, hpfp8_stream_t stream);

/* Small problems.  When a problem has fewer 256 x 256 output tiles than half the GPU's compute units (cfg-1-sized
 * layers, decode-sized M), hpfp8_gemm_per_tensor and hpfp8_gemm_blockwise (sb_gran = 128, no accumulate) run a
 * kernel with 128 x 128 tiles instead, four times as many workgroups; same arithmetic in the same order, identical
 * results.  Test hook, not part of the path: mode 0 = that rule (default), 1 = never, 2 = whenever the form allows
 * (process-wide, stored atomically, takes effect with the next launch). */
void hpfp8_debug_set_small_gemm(int mode);

/* MoE grouped form (one rank's local experts; no counterpart in the reference, whose expert
 * parallelism is unimplemented): rows of a[total_m, K] (row stride lda) are sorted by expert; offs[e] (int32,
 * device) is the inclusive prefix sum of per-expert row counts, a count may be 0, rows past
 * offs[experts-1] are left untouched (an offset below its predecessor or above total_m is read as clamped
 * to that range); b[experts, N, K]; sb[experts, N/128, K/128];
 * sa(m, kb) = sa[m * sa_stride_m + kb * sa_stride_k]; c[total_m, N] bf16 or fp32. */
int hpfp8_gemm_grouped_blockwise(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                                 const void* b, const float* sb, const int32_t* offs, int experts,
                                 int64_t total_m, int64_t N, int64_t K, void* c, int64_t ldc, int out_type,
                                 hpfp8_stream_t stream);

/* The grouped form for power-of-two scales (see hpfp8_gemm_blockwise_pow2); arguments as above. */
int hpfp8_gemm_grouped_blockwise_pow2(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m,
                                      int64_t sa_stride_k, const void* b, const float* sb, const int32_t* offs,
                                      int experts, int64_t total_m, int64_t N, int64_t K, void* c, int64_t ldc,
                                      int out_type, hpfp8_stream_t stream);

/* hpfp8_gemm_grouped_blockwise[_pow2] with the experts' b matrices and scales addressed through strides: expert e's
 * b[N, K] starts b_stride_e bytes after expert e - 1's and has row stride ldb;
 *   sb(e, n, kb) = sb[e * sb_stride_e + (n / 128) * sb_stride_n + kb * sb_stride_k].
 * This is the input gradient of the grouped linear (the dgrad of the same autograd the plain form stands for):
 * with W^T held as the transposed codes [K_w, experts * N_w] that hpfp8_quantize_128x128_bf16 writes for the stacked
 * weight [experts * N_w, K_w] (row stride ld_t), expert e's operand is b + e * N_w with ldb = ld_t, and the
 * weight's scales [experts, N_w / 128, K_w / 128] serve with their two block strides swapped. */
int hpfp8_gemm_grouped_blockwise_strided(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m,
                                         int64_t sa_stride_k, const void* b, int64_t ldb, int64_t b_stride_e,
                                         const float* sb, int64_t sb_stride_e, int64_t sb_stride_n, int64_t sb_stride_k,
                                         const int32_t* offs, int experts, int64_t total_m, int64_t N, int64_t K,
                                         void* c, int64_t ldc, int out_type, int pow2, hpfp8_stream_t stream);

/* ---- MoE grouped weight gradient ----------------------------------------------------------------
 * dW[e] = grad_out_e^T . x_e for every expert e, the contraction running over that expert's own rows
 * [offs[e-1], offs[e]) -- the wgrad of the autograd that hpfp8_gemm_grouped_blockwise stands in for
 * (hyper_parallel/core/shard/_op_dispatch.py:277-283; no grouped counterpart in the reference).  Nothing in this
 * group of calls reads offs on the host, so a grouped backward can be captured in a HIP graph.
 *
 * The 128x1 scaling groups of the two operands run along the tokens and restart at each expert's first row.  The
 * operands therefore live on a padded token axis of hpfp8_grouped_padded_rows(experts, total_m) =
 * (total_m / 128 + experts) * 128 columns: expert e owns max(1, ceil(rows_e / 128)) blocks of 128, the rest of its
 * last block (an empty expert's whole block) holding zero codes.
 *
 *   hpfp8_grouped_layout       offs[experts] (int32, device; read clamped like the grouped GEMM reads it) ->
 *                              layout, hpfp8_grouped_layout_words(experts, total_m) int32 words on the device:
 *                              per expert {first row, rows, first padded block, blocks}, the experts ordered by
 *                              block count, the blocks in use, and the owner of every padded block.
 *   hpfp8_quantize_128x1_t_grouped_bf16
 *                              x[total_m, k] bf16 -> q_t[k, padded] (row stride ld_t bytes >= padded, multiple of 16)
 *                              and scale_inv_t[padded / 128, k] (block-major), expert e's 128-row groups counted
 *                              from its own first row; per expert the same codes and scales as
 *                              hpfp8_quantize_128x1_t_kmajor_bf16 on that expert's rows filled up with zero rows.
 *                              Padded blocks beyond those in use are left untouched.  With q != NULL also the 1x128
 *                              form of the rows that belong to an expert: q[total_m, k], scale_inv[k / 128, total_m]
 *                              (k-block-major), as hpfp8_quantize_1x128_kmajor_bf16 writes them.
 *   hpfp8_gemm_grouped_wgrad   a = grad_out^T codes [N, padded] (row stride lda), sa [padded / 128, N];
 *                              b = x^T codes [K, padded] (row stride ldb), sb [padded / 128, K]; both scale arrays
 *                              contiguous and 16-byte aligned -> c[experts, N, K] contiguous, bf16 or fp32; an
 *                              expert without rows gets zeros.  Per expert the result of hpfp8_gemm_blockwise with
 *                              sb_gran = 1 on that expert's blocks.
 *   hpfp8_grouped_zero_unrouted_rows_bf16
 *                              out[total_m, cols] (row stride ld elements): rows from the last offset on := 0, the rows
 *                              of an input gradient that belong to no expert. */
int64_t hpfp8_grouped_padded_rows(int experts, int64_t total_m);
int64_t hpfp8_grouped_layout_words(int experts, int64_t total_m);
int hpfp8_grouped_layout(const int32_t* offs, int experts, int64_t total_m, int32_t* layout, hpfp8_stream_t stream);
int hpfp8_quantize_128x1_t_grouped_bf16(const void* x, int64_t total_m, int64_t k, const int32_t* layout, int experts,
                                        void* q_t, int64_t ld_t, float* scale_inv_t, void* q, float* scale_inv,
                                        hpfp8_stream_t stream);
int hpfp8_gemm_grouped_wgrad(const void* a, int64_t lda, const float* sa, const void* b, int64_t ldb, const float* sb,
                             const int32_t* layout, int experts, int64_t total_m, int64_t N, int64_t K, void* c,
                             int out_type, hpfp8_stream_t stream);
int hpfp8_grouped_zero_unrouted_rows_bf16(void* out, int64_t ld, const int32_t* offs, int experts, int64_t total_m,
                                          int64_t cols, hpfp8_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HPFP8_H_ */
