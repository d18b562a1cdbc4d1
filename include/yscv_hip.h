/*
 * yscv_hip.h -- C ABI of the MI355X (gfx950) backend for YSCV's quantized-matmul path.
 *
 * The Rust reference exposes this path as plain `pub fn`s over slices
 * (crates/yscv-kernels/src/core.rs:173-186) and has no plugin registry for it, so
 * the drop-in boundary is this function set.  Conventions, modelled on the two
 * native-code precedents in the reference (the `.S` SGEMM kernels declared in
 * crates/yscv-kernels/src/ops/matmul/asm.rs:44-152 and the RKNN matmul context in
 * crates/yscv-kernels/src/rknn/backend.rs:1657-2077):
 *
 *   - every entry point returns an int32 status: 0 = ok, negative = error; the
 *     message of the calling thread's last error is yscv_hip_last_error();
 *   - raw pointers and size_t only, symbol prefix `yscv_hip_`;
 *   - weights live in opaque handles that own device memory and are immutable
 *     after creation, so any number of threads may use one handle concurrently;
 *   - `*_dev` pointers are device addresses and the call is asynchronous on
 *     `stream` (a hipStream_t passed as void*, NULL = the default stream);
 *   - entry points whose names end in `_dispatch`, and every entry point that
 *     takes `_host` pointers, borrow host memory for the duration of the call,
 *     copy in and out themselves and return after the result is in host memory:
 *     these have the exact argument lists of the Rust functions they replace;
 *   - nothing here falls back to CPU arithmetic: a shape a kernel cannot run
 *     is an error (YSCV_HIP_ERR_UNSUPPORTED), never a silent slow path.
 */
#ifndef YSCV_HIP_H
#define YSCV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

#define YSCV_HIP_ABI_VERSION 1u

/* status codes */
#define YSCV_HIP_OK 0
#define YSCV_HIP_ERR_INVALID_ARG (-1) /* shape/pointer contract violated (Rust: debug_assert!) */
#define YSCV_HIP_ERR_DEVICE (-2)      /* a HIP runtime call failed */
#define YSCV_HIP_ERR_OOM (-3)         /* device allocation failed */
#define YSCV_HIP_ERR_UNSUPPORTED (-4) /* valid request this build has no kernel for */
#define YSCV_HIP_ERR_NO_DEVICE (-5)   /* no gfx950 device visible */

/* element types of activations, outputs and scales */
#define YSCV_HIP_F32 0
#define YSCV_HIP_F16 1
#define YSCV_HIP_BF16 2

/* nibble encodings accepted by yscv_hip_int4_weight_create */
#define YSCV_HIP_NIBBLE_SIGNED 0   /* two's complement [-8,7], no zero point: int4_matmul.rs:10-25 */
#define YSCV_HIP_NIBBLE_UNSIGNED 1 /* [0,15] with zero point (default 8): ONNX MatMulNBits */

/* rounding rules of the requantize epilogue */
#define YSCV_HIP_ROUND_HALF_AWAY 0 /* f32::round -- QLinearMatMul, linear.rs:481-485 */
#define YSCV_HIP_ROUND_TIES_EVEN 1 /* round_ties_even -- int8_requant.rs:161-162,550-552 */

/* ---- lifecycle -------------------------------------------------------------- */

/* Select the device (index into the visible HIP devices) and create the
 * library's context.  Idempotent; every other entry point calls it with device 0
 * on first use.  No counterpart in the reference (host_cpu() feature probe,
 * crates/yscv-cpu/src/lib.rs:74-119, plays the same once-per-process role). */
int32_t yscv_hip_init(int32_t device_index);
int32_t yscv_hip_shutdown(void);
uint32_t yscv_hip_abi_version(void);
/* Message of the last error raised on the calling thread ("" if none). */
const char *yscv_hip_last_error(void);
/* Human-readable device / kernel-selection report, like dispatch_report()
 * (crates/yscv-kernels/src/core.rs:79-121).  Writes a NUL-terminated string. */
int32_t yscv_hip_device_info(char *buf, size_t buf_len);

/* Calibration: what this GPU sustains on a plain HBM read stream (1 GiB, GB/s) and on back-to-back matrix
 * instructions held in registers (v_mfma_f32_16x16x32_f16 in TFLOP/s, v_mfma_i32_16x16x64_i8 in TOP/s).  Takes a
 * few milliseconds, allocates 1 GiB for its duration, runs on the default stream.  No counterpart in the reference:
 * its microbenchmark relates the dispatch kernels to its own scalar loops ("SIMD speedup vs scalar",
 * apps/llm-bench/src/bin/kernel_bench.rs:187), not to a machine peak. */
int32_t yscv_hip_measure_peaks(double *hbm_read_gbs, double *mfma_f16_tflops, double *mfma_i8_tops);
/* Calibration of the operand path of the GEMM kernels: GB/s ONE CU takes in through LDS-direct loads
 * (global_load_lds_dwordx4, 1 KiB per wave and instruction, eight in flight per wave, all CUs at once) from a 1 MiB
 * region that every workgroup reads -- it stays in every XCD's L2, so this is the L2 -> CU path alone -- and from a
 * 16 MiB region, more than one XCD's L2 holds.  A tile of (bm + bn) rows needs (bm + bn) * K operand bytes per
 * workgroup whatever the matrix instruction; this figure prices that.  No counterpart in the reference. */
int32_t yscv_hip_measure_fill(double *l2_gbs_per_cu, double *beyond_l2_gbs_per_cu);
/* Calibration: one launch of a kernel that does nothing (one 512-thread workgroup per CU) on `stream`.  A benchmark
 * that times many of them, back to back or as the nodes of a graph, gets the floor under the duration of any kernel
 * (what a single short GEMV cannot go below).  No counterpart in the reference. */
int32_t yscv_hip_launch_empty(void *stream);

/* Device memory helpers for hosts without their own HIP binding. */
int32_t yscv_hip_malloc(void **dev_ptr, size_t bytes);
int32_t yscv_hip_free(void *dev_ptr);
int32_t yscv_hip_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, void *stream);
int32_t yscv_hip_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, void *stream);
int32_t yscv_hip_stream_synchronize(void *stream);

/* ---- packed int4 weights ------------------------------------------------------ */

/* Device-resident form of PackedInt4Weight
 * (crates/yscv-onnx/src/quantize/packed_int4.rs:29-39). */
typedef struct yscv_hip_int4_weight yscv_hip_int4_weight;

/* Upload and re-tile a packed int4 weight.  Host inputs, borrowed:
 *   packed       [n][k/2] bytes, element 2i in the low nibble (int4_matmul.rs:12-14)
 *   scales       [n][k/group_size], scale_dtype F32 or F16
 *   zero_points  NULL, or [n][ceil((k/group_size)/2)] bytes of uint4 (group 2j in the
 *                low nibble) -- only with YSCV_HIP_NIBBLE_UNSIGNED
 * group_size must be even and divide k (int4_matmul.rs:53-54). */
int32_t yscv_hip_int4_weight_create(const uint8_t *packed, const void *scales, int32_t scale_dtype,
                                    const uint8_t *zero_points, int32_t nibble_format, size_t n,
                                    size_t k, size_t group_size, yscv_hip_int4_weight **out);
/* ---- packed int4 weight files -------------------------------------------------
 * The reference keeps PackedInt4Weight in memory only (packed_int4.rs:29-39) and re-quantises the f32 initialisers
 * on every model load (quantize_matmul_weights_int4_packed, packed_int4.rs:50-128); it has no on-disk form.  This
 * one stores exactly the arguments of yscv_hip_int4_weight_create behind a 64-byte header (magic "YSCVI4W", version,
 * dtypes, n, k, group size, FNV-1a 64 checksum; sections padded to 64 bytes), so a quantised weight is uploaded
 * again without the f32 round trip.  write / read_header / read are host-only and need no GPU. */
typedef struct yscv_hip_int4_file_header {
  uint64_t n, k, group_size;
  int32_t scale_dtype, nibble_format, has_zero_points;
  uint64_t packed_bytes, scales_bytes, zero_points_bytes; /* payload sizes the read call expects */
  uint64_t checksum;
} yscv_hip_int4_file_header;
int32_t yscv_hip_int4_file_write(const char *path, const uint8_t *packed, const void *scales, int32_t scale_dtype,
                                 const uint8_t *zero_points, int32_t nibble_format, size_t n, size_t k,
                                 size_t group_size);
/* Validates magic, version, shape contract and that the file length is the one the header implies. */
int32_t yscv_hip_int4_file_read_header(const char *path, yscv_hip_int4_file_header *header);
/* Reads the payload into caller buffers of exactly the header's sizes and verifies the checksum. */
int32_t yscv_hip_int4_file_read(const char *path, uint8_t *packed, size_t packed_bytes, void *scales,
                                size_t scales_bytes, uint8_t *zero_points, size_t zero_points_bytes);
/* read + yscv_hip_int4_weight_create */
int32_t yscv_hip_int4_weight_load(const char *path, yscv_hip_int4_weight **out);

int32_t yscv_hip_int4_weight_destroy(yscv_hip_int4_weight *w);
int32_t yscv_hip_int4_weight_dims(const yscv_hip_int4_weight *w, size_t *n, size_t *k,
                                  size_t *group_size, size_t *device_bytes);

/* y[m][n] = sum_k x[m][k] * W[n][k]; x_dev is [m][k] row-major of x_dtype, y_dev is
 * [m][n] of y_dtype.  `yscv_hip_int4_matmul` picks the kernel from m the way
 * exec_matmul does (crates/yscv-onnx/src/runner/linear.rs:228-278: per-row GEMV
 * below a threshold, GEMM above); `_gemv` forces the skinny kernel (m <= 16,
 * replaces packed_int4_gemv_dispatch, int4_matmul.rs:310-377, called once per row)
 * and `_gemm` the kernels for more rows (replaces packed_int4_gemm_dispatch,
 * int4_matmul.rs:548-605): with 16-bit activations a weight-streaming kernel that keeps all
 * rows' activations in registers up to 32 rows, the LDS-ring MFMA GEMM above. */
int32_t yscv_hip_int4_matmul(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype,
                             void *y_dev, int32_t y_dtype, size_t m, void *stream);
int32_t yscv_hip_int4_gemv(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype,
                           void *y_dev, int32_t y_dtype, size_t m, void *stream);
int32_t yscv_hip_int4_gemm(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype,
                           void *y_dev, int32_t y_dtype, size_t m, void *stream);

/* The int4 matmul with a fused epilogue -- the "bias / residual / activation fusion" the reference plans for its
 * int4 MatMul (docs/int4-quant-pipeline-plan.md:45-51); the decode loop and the prompt pass use exactly these.  Up to
 * 16 rows on the skinny kernel (any activation type); above 16 rows on the kernels for more rows (17 .. 32: the
 * register-resident streaming kernel, more: the LDS-ring MFMA GEMM), fp16 / bf16 activations only (f32 activations
 * with ADD_F32 or SWIGLU above 16 rows: INVALID_ARG).
 *   STORE    y[m][n] = x W^T                       (same as yscv_hip_int4_gemv)
 *   ADD_F32  y[m][n] += x W^T, y_dtype must be F32   (projection + residual add)
 *   SWIGLU   rows 2i / 2i+1 of W are gate_i / up_i; y[m][n/2] = silu(gate) * up   (n even)
 * Results follow the summation order of the kernel that runs, within the int4 tolerance of the unfused call. */
#define YSCV_HIP_EPILOGUE_STORE 0
#define YSCV_HIP_EPILOGUE_ADD_F32 1
#define YSCV_HIP_EPILOGUE_SWIGLU 2
int32_t yscv_hip_int4_matmul_fused(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype,
                                   void *y_dev, int32_t y_dtype, size_t m, int32_t epilogue, void *stream);

/* Same as yscv_hip_int4_matmul, but every byte of device scratch comes from the caller, so
 * the call allocates nothing (the reference allocates its output per call,
 * linear.rs:237; there is no scratch to compare with).  workspace_dev must be 256-byte
 * aligned and at least yscv_hip_int4_workspace_bytes(w, m, x_dtype) long: the prepared
 * activations, the partial sums of the skinny kernel's grid-level K split and, above 16 rows,
 * those of the GEMM's K split (shapes with fewer output tiles than half the CUs); 0 for fp16
 * activations whose K is a multiple of 128 when neither kernel splits K across workgroups. */
int32_t yscv_hip_int4_workspace_bytes(const yscv_hip_int4_weight *w, size_t m, int32_t x_dtype,
                                      size_t *bytes);
int32_t yscv_hip_int4_matmul_ws(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype,
                                void *y_dev, int32_t y_dtype, size_t m, void *workspace_dev,
                                size_t workspace_bytes, void *stream);

/* yscv_hip_int4_matmul for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its kernels need no scratch).  The
 * scratch -- prepared activations and the partial sums of a grid-level K split -- lives in a device array that is
 * part of the library's code object, YSCV_HIP_STATIC_SCRATCH_BYTES per GPU, held until the process ends; the call
 * allocates and frees nothing and enqueues only kernels.  A call whose scratch would exceed that size
 * (yscv_hip_int4_workspace_bytes tells) is YSCV_HIP_ERR_INVALID_ARG; every m <= 16 call fits, and so does a
 * bf16 / fp16 prefill of 2048 x 4096.  All calls on one GPU share the one array: calls that overlap in time (two
 * streams, two threads) race on it -- serialise them, or use yscv_hip_int4_matmul_ws with a workspace per stream.
 * Nothing in the array has to start at zero: every byte a kernel reads was written earlier in the same call.
 * Results are bit-identical to yscv_hip_int4_matmul. */
#define YSCV_HIP_STATIC_SCRATCH_BYTES (32u << 20)
int32_t yscv_hip_int4_matmul_static(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype,
                                    void *y_dev, int32_t y_dtype, size_t m, void *stream);

/* Exact argument lists of the Rust functions (host slices -> host pointers):
 * packed_int4_gemv_dispatch  int4_matmul.rs:310-318
 * packed_int4_gemm_dispatch  int4_matmul.rs:548-557
 * pack_int4_symmetric_per_group  int4_matmul.rs:611-616 (returns into caller buffers
 *   packed_out[m_w*k/2], scales_out[m_w*k/group_size])
 * dequantize_int4_to_f32     ops/quantize.rs:18 (output[2*n_bytes])
 * quantize_f32_to_int4       ops/quantize.rs:69 (output[(len+1)/2]: q = clamp(round_ties_even(x / scale) + zp, -8, 7),
 *   element 2i in the low nibble, |scale| <= f32::EPSILON quantises everything to zp); `_dev` is the same on device
 *   pointers, asynchronous on `stream` */
int32_t yscv_hip_packed_int4_gemv_dispatch(const uint8_t *weight_packed, const float *scales,
                                           const float *activation, float *output, size_t m_w,
                                           size_t k, size_t group_size);
int32_t yscv_hip_packed_int4_gemm_dispatch(const uint8_t *weight_packed, const float *scales,
                                           const float *activation, float *output, size_t m,
                                           size_t n, size_t k, size_t group_size);
int32_t yscv_hip_pack_int4_symmetric_per_group(const float *weights, size_t m_w, size_t k,
                                               size_t group_size, uint8_t *packed_out,
                                               float *scales_out);
int32_t yscv_hip_dequantize_int4_to_f32(const uint8_t *packed, size_t n_bytes, float scale,
                                        int8_t zero_point, float *output);
int32_t yscv_hip_quantize_f32_to_int4(const float *data, size_t len, float scale, int8_t zero_point,
                                      uint8_t *output);
int32_t yscv_hip_quantize_f32_to_int4_dev(const float *data_dev, size_t len, float scale, int8_t zero_point,
                                          uint8_t *out_dev, void *stream);

/* ---- int8 GEMM ------------------------------------------------------------------ */

/* Device-resident form of PackedI8B (crates/yscv-kernels/src/ops/int8_matmul.rs:128-160):
 * B re-tiled for the MFMA kernel plus its per-column sums. */
typedef struct yscv_hip_i8_weight yscv_hip_i8_weight;

/* pack_i8_b_for_matmul (int8_matmul.rs:163): b_host is row-major [k][n]. */
int32_t yscv_hip_pack_i8_b_for_matmul(const int8_t *b_host, size_t k, size_t n,
                                      yscv_hip_i8_weight **out);
int32_t yscv_hip_i8_weight_destroy(yscv_hip_i8_weight *b);
int32_t yscv_hip_i8_weight_dims(const yscv_hip_i8_weight *b, size_t *k, size_t *n);

/* out[i][j] = sum_k (a[i][k] - a_zp) * b[k][j] in exact int32.
 * a_dev is [m][k]; a_is_u8 = 0: int8 activations (then a_zp is usually 0, the
 * int8_matmul_prepacked_dispatch contract, int8_matmul.rs:2420); a_is_u8 = 1: uint8
 * activations with zero point a_zp (MatMulInteger, ONNX).  The zero point is folded as
 * acc - a_zp * colsum(b), the algebra of
 * crates/yscv-onnx/src/runner/conv/quantized.rs:119-147. */
int32_t yscv_hip_int8_matmul(const void *a_dev, int32_t a_is_u8, int32_t a_zp,
                             const yscv_hip_i8_weight *b, size_t m, int32_t *out_dev, void *stream);

/* Same GEMM with the requantize epilogue fused (no int32 round trip through HBM):
 *   q = clamp(round(f32(acc + corr[j]) * composite[j] + y_zp), clamp_lo, clamp_hi)
 * corr_dev / composite_dev are per-column device arrays or NULL (then corr = 0 and
 * the scalar `composite` is used).  round_mode HALF_AWAY with [-128,127] is the
 * QLinearMatMul fast path (linear.rs:481-485); TIES_EVEN is
 * requant_i8_per_channel_dispatch (int8_requant.rs:401-429).  out_dev is [m][n] bytes:
 * int8 when clamp_lo < 0, otherwise uint8 (range [0,255] is an extension: the
 * reference always clamps to [-128,127], linear.rs:484). */
int32_t yscv_hip_int8_matmul_requant(const void *a_dev, int32_t a_is_u8, int32_t a_zp,
                                     const yscv_hip_i8_weight *b, size_t m,
                                     const int32_t *corr_dev, const float *composite_dev,
                                     float composite, float y_zp, int32_t round_mode,
                                     int32_t clamp_lo, int32_t clamp_hi, void *out_dev,
                                     void *stream);

/* Exact argument lists of int8_matmul_dispatch (int8_matmul.rs:2407; b is [k][n]) and
 * int8_matmul_prepacked_dispatch (int8_matmul.rs:2420), host pointers. */
int32_t yscv_hip_int8_matmul_dispatch(const int8_t *a, const int8_t *b, size_t m, size_t k,
                                      size_t n, int32_t *out);
int32_t yscv_hip_int8_matmul_prepacked_dispatch(const int8_t *a, const yscv_hip_i8_weight *b,
                                                size_t m, int32_t *out);

/* ---- quantize / requantize / DynamicQuantizeLinear (device pointers) -------------- */

/* quantize_linear_f32_to_i8_dispatch (ops/quantize.rs:154):
 * q = clamp(round_ties_even(v / scale + zero_point), -128, 127). */
int32_t yscv_hip_quantize_linear_f32_to_i8(const float *data_dev, size_t len, float scale,
                                           float zero_point, int8_t *out_dev, void *stream);
/* requant_i8_per_channel_dispatch (ops/int8_requant.rs:401): acc is [len/c][c]. */
int32_t yscv_hip_requant_i8_per_channel(const int32_t *acc_dev, size_t len,
                                        const int32_t *corr_dev, const float *composite_dev,
                                        float y_zp, int8_t *out_dev, size_t c, void *stream);
/* requant_i32_row_to_i8_dispatch (ops/int8_requant.rs:81): bias_dev may be NULL. */
int32_t yscv_hip_requant_i32_row_to_i8(const int32_t *acc_dev, size_t len, const int32_t *bias_dev,
                                       float composite, float y_zp, int32_t relu, int8_t *out_dev,
                                       size_t c, void *stream);
/* exec_dynamic_quantize_linear (crates/yscv-onnx/src/runner/misc.rs:241-289):
 * y_dev[len] uint8, scale_zp_dev[0] = scale, scale_zp_dev[1] = zero point (as f32). */
int32_t yscv_hip_dynamic_quantize_linear(const float *x_dev, size_t len, uint8_t *y_dev,
                                         float *scale_zp_dev, void *stream);

/* Host-pointer forms with the Rust argument lists. */
int32_t yscv_hip_quantize_linear_f32_to_i8_dispatch(const float *data, size_t len, float scale,
                                                    float zero_point, int8_t *output);
int32_t yscv_hip_requant_i8_per_channel_dispatch(const int32_t *acc, size_t len,
                                                 const int32_t *corr, const float *composite,
                                                 float y_zp, int8_t *out, size_t c);
int32_t yscv_hip_requant_i32_row_to_i8_dispatch(const int32_t *acc, size_t len,
                                                const int32_t *bias, float composite, float y_zp,
                                                int32_t relu, int8_t *out, size_t c);
int32_t yscv_hip_dynamic_quantize_linear_host(const float *x, size_t len, uint8_t *y,
                                              float *scale, float *zero_point);

/* ---- ONNX operators on f32 carriers (device pointers) ------------------------------------- */

/* The reference runner keeps every quantised tensor as f32 values holding integers; these entry points
 * take and return such tensors in device memory, so a graph executor calls them where the reference
 * calls the function cited.  Operands are rank 2 (callers flatten leading dimensions of A into m). */

/* Which route a call took (written to *path_out when it is not null). */
#define YSCV_HIP_PATH_FAST 0            /* both zero points 0: integer kernel, as the reference's fast path */
#define YSCV_HIP_PATH_FALLBACK_EXACT 1  /* non-zero zero point, 8-bit integer operands: exact integer route */
#define YSCV_HIP_PATH_FALLBACK_F32 2    /* non-zero zero point, other operands: f32 products added in k order */

/* QuantRuntimeStats (crates/yscv-onnx/src/runner/quant_stats.rs:6-22) restricted to this path, plus the
 * int4_fast / int4_fallback split docs/int4-quant-pipeline-plan.md:25-34 asks a runtime to report and the
 * same split for MatMulInteger.  "fallback" counts every call the reference would send to its f32 matmul
 * (linear.rs:494), whichever device route served it here.  int4_fast counts calls served by the tiled MFMA
 * kernels, int4_fallback calls served by the generic per-group kernel. */
typedef struct yscv_hip_quant_stats {
  uint64_t qlinear_matmul_fast;
  uint64_t qlinear_matmul_fallback;
  uint64_t matmul_integer_fast;
  uint64_t matmul_integer_fallback;
  uint64_t int4_fast;
  uint64_t int4_fallback;
} yscv_hip_quant_stats;
/* quant_runtime_stats / reset_quant_runtime_stats (quant_stats.rs:24-62): process-wide, relaxed atomics. */
int32_t yscv_hip_quant_runtime_stats(yscv_hip_quant_stats *out);
int32_t yscv_hip_reset_quant_runtime_stats(void);
/* quant_int8_fast_enabled (quant_stats.rs:64-69): 0 only when YSCV_QUANT_INT8_FAST is exactly "0". */
int32_t yscv_hip_quant_int8_fast_enabled(void);
/* should_use_prepacked_i8_b (crates/yscv-onnx/src/runner/layout.rs:6-11) and the load-time gate
 * should_prepack_i8_b (crates/yscv-onnx/src/plan/build.rs:1371-1377); 1 = yes. */
int32_t yscv_hip_should_use_prepacked_i8_b(size_t m, size_t k, size_t n);
int32_t yscv_hip_should_prepack_i8_b(size_t k, size_t n);
/* Load-time prepack of a weight initialiser held as an f32 carrier [k][n] on the device: `v.round() as i8`
 * per element (tensor_data_as_i8, plan/build.rs:1367-1369), then the layout of
 * yscv_hip_pack_i8_b_for_matmul (plan/build.rs:1416-1454). */
int32_t yscv_hip_i8_weight_from_f32(const float *b_dev, size_t k, size_t n, void *stream,
                                    yscv_hip_i8_weight **out);
/* exec_matmul_integer (crates/yscv-onnx/src/runner/linear.rs:648-737).  out_dev[m][n] f32.  Pass the
 * unpacked B (b_dev, [k][n]), a prepacked one, or both; absent ONNX zero points are 0.  A prepacked B
 * alone serves b_zp == 0 only. */
int32_t yscv_hip_exec_matmul_integer(const float *a_dev, const float *b_dev,
                                     const yscv_hip_i8_weight *b_packed, float a_zp, float b_zp, size_t m,
                                     size_t k, size_t n, float *out_dev, int32_t *path_out, void *stream);
/* exec_qlinear_matmul (crates/yscv-onnx/src/runner/linear.rs:438-538): scalar scales and zero points,
 * output clamp(round_half_away(.), -128, 127) as f32.  A prepacked B whose shape differs from (k, n) is
 * an error, as in the reference (linear.rs:468-475). */
int32_t yscv_hip_exec_qlinear_matmul(const float *a_dev, float a_scale, float a_zp, const float *b_dev,
                                     const yscv_hip_i8_weight *b_packed, float b_scale, float b_zp,
                                     float y_scale, float y_zp, size_t m, size_t k, size_t n,
                                     float *out_dev, int32_t *path_out, void *stream);
/* The triple the reference's rewriter emits for a quantised MatMul, QuantizeLinear -> QLinearMatMul ->
 * DequantizeLinear with symmetric activations and weights (crates/yscv-onnx/src/quantize/rewriter.rs:586-673), as
 * one call on f32 in / f32 out: a_q = clamp(round_ties_even(x / a_scale), -128, 127) (misc.rs:42-80), the int8
 * product against the prepacked weight, q = clamp(round_half_away(acc * ((a_scale * b_scale) / y_scale) + y_zp),
 * -128, 127) (linear.rs:481-485), y = (q - y_zp) * y_scale (misc.rs:124-128).  Bit-identical to running the three
 * operators one after the other; counted as one qlinear_matmul_fast. */
int32_t yscv_hip_exec_qdq_matmul(const float *x_dev, size_t m, float a_scale, const yscv_hip_i8_weight *b,
                                 float b_scale, float y_scale, float y_zp, float *out_dev, void *stream);
/* DynamicQuantizeLinear feeding MatMulInteger, the pair ONNX Runtime's dynamic quantisation emits (exec_dynamic_quantize_linear,
 * crates/yscv-onnx/src/runner/misc.rs:241-289, then exec_matmul_integer with a_zero_point = the y_zero_point just computed,
 * runner/linear.rs:648-737), as one call: x_dev [m][k] f32 is reduced to its range, quantised to uint8 once into
 * stream-ordered scratch, and multiplied against the prepacked int8 weight (b_zero_point 0); the zero point never leaves
 * the device (the GEMM's epilogue reads it there and folds (128 - zp) * colsum(b)), the f32 carriers of the quantised
 * activations are never written, no range scan and no host synchronisation.  out_dev [m][n] = f32 of the exact integer sum
 * of (a_q - zp) * b; *y_scale_dev, *y_zp_dev as DynamicQuantizeLinear returns them.  Bit-identical to the two operators
 * called one after the other.  Counted as matmul_integer_fallback (a non-zero a_zero_point sends the reference to its
 * f32 matmul, linear.rs:701-736). */
int32_t yscv_hip_exec_dql_matmul_integer(const float *x_dev, size_t m, const yscv_hip_i8_weight *b, float *out_dev,
                                         float *y_scale_dev, float *y_zp_dev, void *stream);
/* MatMulNBits (com.microsoft), the operator ONNX exporters emit for 4-bit weights: Y = A x dequant(B)^T + bias.  The
 * reference's dispatcher has no such operator (crates/yscv-onnx/src/runner/dispatch.rs:191-322), so its int4 branch
 * only ever sees weights it packed itself; here the initialisers of the node -- B [N][K/block][block/2] bytes, element
 * 2i in the low nibble (the byte order of PackedInt4Weight, int4_matmul.rs:12-14), scales [N*K/block] f32 or f16,
 * optional packed uint4 zero_points [N][ceil(K/block/2)], default 8 -- are uploaded once with
 * yscv_hip_int4_weight_create(B, scales, dtype, zero_points, YSCV_HIP_NIBBLE_UNSIGNED, N, K, block) at load time, and
 * the executor passes the node's attributes, which must agree with the handle (a mismatch is the runner's ShapeMismatch
 * error; bits other than 4 is unsupported; g_idx is not supported).  a_dev is [m][K] with the leading dimensions of A
 * flattened into m, bias_dev is null or [N] f32; with a bias the f32 product plus bias is rounded once to y_dtype.
 * Kernel choice by m as in yscv_hip_int4_matmul; counted in int4_fast / int4_fallback. */
int32_t yscv_hip_exec_matmul_nbits(const void *a_dev, int32_t a_dtype, size_t m, const yscv_hip_int4_weight *b,
                                   const float *bias_dev, int64_t attr_k, int64_t attr_n, int64_t attr_bits,
                                   int64_t attr_block_size, void *y_dev, int32_t y_dtype, void *stream);
/* Gemm whose weight the int4 packing pass quantised (quantize_matmul_weights_int4_packed packs Gemm weights for both
 * transB values, crates/yscv-onnx/src/quantize/packed_int4.rs:155-168, but exec_gemm never reads them,
 * runner/linear.rs:5,228): Y = alpha * (A x W^T) + beta * C on f32 carriers with the int4 product in place of the f32
 * one.  W is the handle yscv_hip_int4_weight_from_f32 made from the Gemm's B (either layout), a_dev is [m][K] (a transA
 * node is transposed by the caller, as exec_gemm does first), c_dev is null (c_rows 0), one row of N values broadcast over
 * the rows (c_rows 1) or [m][N] (c_rows m).  alpha and beta are applied only when they differ from 1 by more than
 * f32::EPSILON, each as its own rounded multiply before the rounded add, like Tensor::scale + kernel_add
 * (linear.rs:54-66). */
int32_t yscv_hip_exec_gemm_int4(const float *a_dev, size_t m, const yscv_hip_int4_weight *b, const float *c_dev,
                                size_t c_rows, float alpha, float beta, float *y_dev, void *stream);
/* exec_quantize_linear, f32-carrier arm (crates/yscv-onnx/src/runner/misc.rs:42-80) =
 * quantize_linear_f32_to_f32_i8_scalar (crates/yscv-kernels/src/ops/quantize.rs:226-238). */
int32_t yscv_hip_exec_quantize_linear(const float *x_dev, size_t len, float scale, float zero_point,
                                      float *out_dev, void *stream);
/* exec_dequantize_linear (crates/yscv-onnx/src/runner/misc.rs:110-239) on a tensor viewed as
 * [outer][chan][inner] around the quantisation axis.  n_scales = 1: per tensor; n_scales = chan: per
 * channel; anything else is the reference's "scale len" error.  zps_dev may be null (all zero). */
int32_t yscv_hip_exec_dequantize_linear(const float *q_dev, size_t outer, size_t chan, size_t inner,
                                        const float *scales_dev, const float *zps_dev, size_t n_scales,
                                        float *out_dev, void *stream);
/* exec_dynamic_quantize_linear (crates/yscv-onnx/src/runner/misc.rs:241-289) with its three f32 outputs:
 * y_dev[len], *y_scale_dev, *y_zp_dev. */
int32_t yscv_hip_exec_dynamic_quantize_linear(const float *x_dev, size_t len, float *y_dev,
                                              float *y_scale_dev, float *y_zp_dev, void *stream);

/* quantize_matmul_weights_int4_packed (crates/yscv-onnx/src/quantize/packed_int4.rs:50-128) for one weight
 * initialiser held as f32 on the device.  layout KN: shape [d0 = K][d1 = N] (MatMul, Gemm transB = 0), transposed
 * before packing; layout NK: shape [d0 = N][d1 = K] (Gemm transB = 1), packed as it is.  Symmetric per-group
 * packing (pack_int4_symmetric_per_group, int4_matmul.rs:611-646), f32 scales.  group_size 0 or odd is the
 * reference's error; a weight the reference skips (K % group_size != 0 or K * N < 32) returns OK with *out = NULL. */
#define YSCV_HIP_WEIGHT_KN 0
#define YSCV_HIP_WEIGHT_NK 1
int32_t yscv_hip_int4_weight_from_f32(const float *w_dev, size_t d0, size_t d1, int32_t layout, size_t group_size,
                                      void *stream, yscv_hip_int4_weight **out);

/* KvCache int8 storage (crates/yscv-onnx/src/runner/kv_cache.rs:45-61): per-row symmetric int8 of the rows being
 * appended, src_dev[rows][kv_dim] f32 -> data_dev[rows][kv_dim] int8 + scales_dev[rows]; and the read side
 * (dequantise_to_vec, kv_cache.rs:64-79). */
int32_t yscv_hip_kv_i8_quantize_rows(const float *src_dev, size_t rows, size_t kv_dim, int8_t *data_dev,
                                     float *scales_dev, void *stream);
int32_t yscv_hip_kv_i8_dequantize_rows(const int8_t *data_dev, const float *scales_dev, size_t rows, size_t kv_dim,
                                       float *out_dev, void *stream);

/* ---- the operators between the MatMuls of an LLM graph, on device tensors ------------------------------------
 * A graph executor that keeps its tensors on the GPU calls these between two projections instead of leaving the
 * device; layouts and arithmetic are the reference operators', f32 in and out. */
/* rms_norm_last_dim (crates/yscv-kernels/src/ops/norm.rs:1431-1518): y[row] = x[row] * (1 / sqrt(mean(x[row]^2) + eps))
 * * gamma over rows of d values; epsilon must be finite and > 0 (InvalidRmsNormEpsilon -> INVALID_ARG). */
int32_t yscv_hip_rms_norm_dev(const float *x_dev, const float *gamma_dev, size_t rows, size_t d, float eps, float *y_dev,
                              void *stream);
/* apply_rotary_embedding (crates/yscv-kernels/src/ops/rope.rs:24-117), in place: q [seq_len][num_q_heads][d_head],
 * k [seq_len][num_kv_heads][d_head], pair (x[i], x[i + d/2]) rotated by inv_freq[i] * (pos + seq_offset) with
 * inv_freq[i] = 1 / theta^(2i / d_head).  sin / cos come from the device's math library: tolerance, not bit parity. */
int32_t yscv_hip_rope_dev(float *q_dev, float *k_dev, size_t num_q_heads, size_t num_kv_heads, size_t d_head, size_t seq_len,
                          size_t seq_offset, float theta, void *stream);
/* exec_grouped_query_attention (crates/yscv-onnx/src/runner/linear.rs:552-646): q [batch][seq_q][num_q_heads * d_head],
 * k / v [batch][seq_k][num_kv_heads * d_head] -> out [batch][seq_q][num_q_heads * d_head]; kv head = q head / groups,
 * scores * 1 / sqrt(d_head), max-subtracted softmax over all seq_k positions, no mask.  d_head 32, 64, 96 or 128
 * (UNSUPPORTED otherwise); operands enter the matrix cores as fp16 with f32 accumulation (relative error about 1e-3).
 * q, k and out must be 16-byte aligned. */
int32_t yscv_hip_gqa_attention_dev(const float *q_dev, const float *k_dev, const float *v_dev, size_t batch, size_t seq_q,
                                   size_t seq_k, size_t num_q_heads, size_t num_kv_heads, size_t d_head, float *out_dev,
                                   void *stream);

/* ---- decode loop (Llama-style decoder, int4 projections, fp16 KV cache) ----------------- */

/* GPU-resident counterpart of the llm-bench decode loop (apps/llm-bench/src/main.rs:403-561:
 * feed the last token and the KV cache, greedy pick, repeat), of KvCache
 * (crates/yscv-onnx/src/runner/kv_cache.rs:14-254) and of greedy generate()
 * (crates/yscv-onnx/src/generate.rs:58-208, top_k = 1).  Every linear layer goes through the
 * skinny int4 kernel; q/k/v and gate/up are fused into one weight each at finalize time. */
typedef struct yscv_hip_decoder yscv_hip_decoder;

typedef struct yscv_hip_decoder_config {
  int32_t n_layers;
  int32_t d_model;
  int32_t n_heads;    /* query heads */
  int32_t n_kv_heads; /* divides n_heads; head_dim 128 with 1..4 query heads per kv head takes the specialised
                         attention kernels (fp16 or int8 cache, single-launch path), anything else the general one */
  int32_t head_dim;   /* 32, 64, 96 or 128 */
  int32_t d_ff;
  int32_t vocab;
  int32_t group_size; /* int4 group size of every projection: 32, 64 or a multiple of 128 */
  int32_t max_batch;  /* 1..16 */
  int32_t max_ctx;    /* KV cache capacity in positions, multiple of 128 */
  int32_t max_steps;  /* capacity of the generated-token history */
  float rope_theta;
  float rms_eps;
} yscv_hip_decoder_config;

/* projection kinds for yscv_hip_decoder_set_linear */
#define YSCV_HIP_DEC_Q 0
#define YSCV_HIP_DEC_K 1
#define YSCV_HIP_DEC_V 2
#define YSCV_HIP_DEC_O 3
#define YSCV_HIP_DEC_GATE 4
#define YSCV_HIP_DEC_UP 5
#define YSCV_HIP_DEC_DOWN 6
#define YSCV_HIP_DEC_LM_HEAD 7
/* norm kinds for yscv_hip_decoder_set_norm */
#define YSCV_HIP_DEC_ATTN_NORM 0
#define YSCV_HIP_DEC_FFN_NORM 1
#define YSCV_HIP_DEC_FINAL_NORM 2

int32_t yscv_hip_decoder_create(const yscv_hip_decoder_config *cfg, yscv_hip_decoder **out);
/* The same with the storage type of the KV cache chosen (llm-bench --kv-dtype, apps/llm-bench/src/main.rs:232-265;
 * KvCache::with_dtype, crates/yscv-onnx/src/runner/kv_cache.rs:14-61).  I8: every appended K row and V row (the
 * kv_dim = n_kv_heads * head_dim values of one position) is stored as int8 with one f32 scale, scale = absmax / 127
 * (1.0 when absmax <= f32::EPSILON), q = clamp(round_half_away(v / scale), -127, 127), and attention reads q * scale;
 * the current token attends to its own quantised row, as the reference's loop appends before it reads.  Half the
 * cache bytes of fp16 per step.  Multi-kernel path only (use_graph 0 or 1). */
#define YSCV_HIP_KV_F16 0
#define YSCV_HIP_KV_I8 1
int32_t yscv_hip_decoder_create_kv(const yscv_hip_decoder_config *cfg, int32_t kv_dtype, yscv_hip_decoder **out);
int32_t yscv_hip_decoder_destroy(yscv_hip_decoder *d);
/* Host inputs, borrowed: packed [n][k/2] uint4 nibbles (zero point 8, MatMulNBits order),
 * scales_f16 [n][k/group_size] fp16 bit patterns.  `layer` is ignored for LM_HEAD. */
int32_t yscv_hip_decoder_set_linear(yscv_hip_decoder *d, int32_t layer, int32_t kind,
                                    const uint8_t *packed, const uint16_t *scales_f16, size_t n,
                                    size_t k);
int32_t yscv_hip_decoder_set_norm(yscv_hip_decoder *d, int32_t layer, int32_t kind,
                                  const float *gamma);
int32_t yscv_hip_decoder_set_embedding(yscv_hip_decoder *d, const uint16_t *table_f16);
/* Build the fused device weights from what was set; required before run. */
int32_t yscv_hip_decoder_finalize(yscv_hip_decoder *d);
/* Benchmark setup: random-initialised weights of the configured architecture generated on the
 * device (uniform nibbles, scales ~U(0.005,0.02), embedding ~N(0,1)), and a KV cache filled with
 * ~N(0,1) values.  No reference counterpart (llm-bench loads an ONNX file). */
int32_t yscv_hip_decoder_init_random(yscv_hip_decoder *d, uint64_t seed);
/* The same with the nibbles uniform over nibble_lo .. nibble_hi.  0 .. 15 has mean -0.5 after the zero point 8,
 * which gives every projection output a common offset and makes a deep random model ill-conditioned (all logits
 * nearly equal); 1 .. 15 is symmetric about the zero point and yields a model whose greedy tokens vary. */
int32_t yscv_hip_decoder_init_random_range(yscv_hip_decoder *d, uint64_t seed, int32_t nibble_lo,
                                           int32_t nibble_hi);
int32_t yscv_hip_decoder_fill_kv_random(yscv_hip_decoder *d, uint64_t seed);
/* Load cache positions [0, n_positions) of one layer from host arrays laid out
 * [batch][position][kv_head][head_dim] fp16 (keys already rotated). */
int32_t yscv_hip_decoder_set_kv(yscv_hip_decoder *d, int32_t layer, const uint16_t *k_f16,
                                const uint16_t *v_f16, int32_t batch, int32_t n_positions);
/* The read side of the cache (KvCache::get, crates/yscv-onnx/src/runner/kv_cache.rs:207-241): positions
 * [first_pos, first_pos + n_positions) of one layer into host arrays laid out like yscv_hip_decoder_set_kv's,
 * [batch][position][kv_head][head_dim] fp16, keys as stored (rotated). */
int32_t yscv_hip_decoder_get_kv(yscv_hip_decoder *d, int32_t layer, uint16_t *k_f16, uint16_t *v_f16,
                                int32_t batch, int32_t first_pos, int32_t n_positions);
/* Start a generation: batch rows, the position the next token is written at, one input token per row. */
int32_t yscv_hip_decoder_reset(yscv_hip_decoder *d, int32_t batch, int32_t start_pos,
                               const int32_t *tokens_host);
/* Run n_steps decode steps (asynchronously on `stream`).  use_graph = 0 launches the kernels of a step one
 * by one, 1 replays one captured HIP graph per step, 2 runs all n_steps in ONE cooperative launch of the
 * persistent decode kernel (batch 1 only; YSCV_HIP_ERR_UNSUPPORTED with the reason in the error text when
 * the model shape or the device cannot run it), YSCV_HIP_DECODE_AUTO picks 2 where it applies (batch 1, fp16
 * cache, supported shape) and 1 otherwise.  Paths 0 and 1 run the same kernels and give the same bits; path 2
 * rounds its fp16 activations at other points, so its logits agree with theirs to about 1e-4 .. 5e-3 of max|logit|
 * (each path is within the float bar of the int4 kernels against the reference arithmetic) and a greedy pick can
 * differ where two logits are that close.  A caller that needs one arithmetic for every batch size names the path
 * instead of passing AUTO; yscv_hip_decoder_last_path tells which one a call took.  Fails if the KV cache or the
 * token history would overflow (KvCache::append returns an error in the same situation, kv_cache.rs:160-185). */
#define YSCV_HIP_DECODE_AUTO 3
int32_t yscv_hip_decoder_run(yscv_hip_decoder *d, int32_t n_steps, int32_t use_graph, void *stream);
/* The prompt phase of the decode loop (apps/llm-bench/src/main.rs:403-470 times it apart from the decode phase): feeds
 * n_tokens prompt tokens at positions start_pos .. start_pos + n_tokens - 1 of batch row 0 in ONE pass -- every
 * projection sees all rows at once (the MFMA GEMM above 16 rows), attention is causal over the cache, which receives
 * the rotated keys and the values of every position -- and computes the logits of the last position only.  Leaves the
 * decoder as yscv_hip_decoder_reset(1, start_pos + n_tokens - 1, last token) + one decode step would: batch 1, the
 * greedy pick as the next input token and as token 0 of the history, position start_pos + n_tokens, step 1.  The
 * results agree with token-by-token feeding to the float bar of the int4 kernels (the GEMM folds the group scale into
 * fp16 weights where the decode kernel applies it in fp32).  With an int8 cache every row is quantised as the decode
 * step quantises it (scales over all kv heads of the position) and attention reads what the cache returns for each
 * position, q * scale of its row, earlier positions included.  tokens_host is read before the call returns. */
int32_t yscv_hip_decoder_prefill(yscv_hip_decoder *d, const int32_t *tokens_host, int32_t n_tokens, int32_t start_pos,
                                 void *stream);
/* Rows of the prompt that yscv_hip_decoder_prefill takes through the layers in one pass (default 4096).  A longer
 * prompt runs as several passes, each appending to the cache the earlier ones wrote; the per-call scratch (activations of
 * one pass: rows x (3 d_model + q/k/v width + n_heads head_dim + d_ff) x 2 bytes and up) scales with this number, the
 * results do not depend on it beyond the float tolerance.  No counterpart in the reference (its prompt phase feeds
 * the whole prompt at once, apps/llm-bench/src/main.rs:403-470). */
int32_t yscv_hip_decoder_set_prefill_rows(yscv_hip_decoder *d, int32_t rows);
/* Optional bias of the fused q / k / v projection of one layer (Qwen-style attention; the reference adds it with
 * the Add node behind the MatMul): fp16 [(n_heads + 2 n_kv_heads) * head_dim] in q, k, v order, or NULL to remove it.
 * A decoder with a bias takes the multi-kernel path (the single-launch kernel has none). */
int32_t yscv_hip_decoder_set_qkv_bias(yscv_hip_decoder *d, int32_t layer, const uint16_t *bias_f16);
/* The path the last yscv_hip_decoder_run of this decoder took: 0, 1 or 2 as above, -1 before the first call.
 * (The reference has one CPU path and no counterpart; this is how a caller of AUTO learns what ran.) */
int32_t yscv_hip_decoder_last_path(const yscv_hip_decoder *d, int32_t *path);
/* Measurement aid: enqueue only the int4 projections of n_steps decode steps (same weights, same
 * order, same buffers as a real step, no attention / norm / sampling), so that the projections'
 * share of a step can be timed on its own.  The activations it reads are whatever the buffers hold. */
int32_t yscv_hip_decoder_run_projections(yscv_hip_decoder *d, int32_t n_steps, void *stream);
/* Generated tokens of steps [first_step, first_step + n_steps), laid out [step][batch]. */
int32_t yscv_hip_decoder_read_tokens(yscv_hip_decoder *d, int32_t first_step, int32_t n_steps,
                                     int32_t *out_host);
/* Logits of the last step, [batch][vocab] f32. */
int32_t yscv_hip_decoder_read_logits(yscv_hip_decoder *d, float *out_host);
/* Inspection aid for parity tests: the activation buffers of the multi-kernel path (use_graph 0 or 1) as the last
 * step left them, widened to f32, [batch][width]: the residual stream after the last layer, the final RMSNorm's
 * output (the LM head's input), and the last layer's q|k|v (q and k rotated), attention output and SwiGLU output.
 * The single-launch path keeps these in registers and exchange records and does not fill them.  No counterpart in
 * the reference (its runner keeps every intermediate tensor in the TensorEnv by name). */
#define YSCV_HIP_DEC_ACT_RESIDUAL 0 /* [batch][d_model] */
#define YSCV_HIP_DEC_ACT_NORMED 1   /* [batch][d_model] */
#define YSCV_HIP_DEC_ACT_QKV 2      /* [batch][(n_heads + 2 n_kv_heads) * head_dim] */
#define YSCV_HIP_DEC_ACT_ATTN_OUT 3 /* [batch][n_heads * head_dim] */
#define YSCV_HIP_DEC_ACT_FFN 4      /* [batch][d_ff] */
int32_t yscv_hip_decoder_read_activation(yscv_hip_decoder *d, int32_t which, float *out_host, size_t capacity);
/* Test aid: the single-launch path stamps what its workgroups hand to each other with a 24-bit tag that advances with
 * every step; close to the end of the tag space yscv_hip_decoder_run clears the exchange buffers and starts the count
 * again.  This sets the count (>= 1), so that a test reaches that point without half a million decode steps. */
int32_t yscv_hip_decoder_debug_set_tag_epoch(yscv_hip_decoder *d, uint32_t epoch);
/* Test aid: the multi-kernel path runs rotary embedding and cache append (fp16 or int8) inside the attention kernel;
 * 0 switches to the separate rope_append launch in front of it, which computes the same values, so that a test can hold
 * one against the other.  Drops a captured graph.  No counterpart in the reference. */
int32_t yscv_hip_decoder_debug_set_fused_attention(yscv_hip_decoder *d, int32_t on);
/* Test aid: the multi-kernel path folds every RMSNorm into the projections around it when the shapes allow (the
 * kernel that updates the residual stream also writes fp16(h * gamma * p), p a power of two per row near
 * 1 / (4 rms) of the row before the update, and per-row partial sums of h^2; the projection that follows applies
 * 1 / (p * sqrt(mean(h^2) + eps)) to its sums); 0 switches back to RMSNorm as a launch of
 * its own, so that a test can hold one against the other (same product, the fp16 rounding taken before the row factor
 * instead of after it).  Drops a captured graph.  No counterpart in the reference. */
int32_t yscv_hip_decoder_debug_set_folded_norm(yscv_hip_decoder *d, int32_t on);
/* Bytes of packed weights + scales one decode step streams through the projections. */
int32_t yscv_hip_decoder_weight_bytes(const yscv_hip_decoder *d, size_t *bytes);
int32_t yscv_hip_decoder_vocab(const yscv_hip_decoder *d, size_t *vocab);

/* GenerateConfig (crates/yscv-onnx/src/generate.rs:9-35; its Default is 256, 1.0, 50, 0.9, no EOS, 1.0). */
typedef struct yscv_hip_generate_config {
  size_t max_tokens;
  float temperature;        /* 1.0 = unchanged; values <= 0 are ignored like in the reference */
  size_t top_k;             /* 0 = disabled; 1 = greedy */
  float top_p;              /* 1.0 = disabled */
  int32_t has_eos;          /* Option<u32>: 0 = None */
  uint32_t eos_token_id;
  float repetition_penalty; /* 1.0 = disabled */
} yscv_hip_generate_config;
/* sample_token (generate.rs:121-208) on host logits, in place: top-k threshold, softmax, top-p cut, xorshift64
 * draw; *rng is the sampler state (generate() starts it at 0xdeadbeef). */
int32_t yscv_hip_sample_token(float *logits, size_t vocab_size, size_t top_k, float top_p, uint64_t *rng,
                              uint32_t *token_out);
/* generate (generate.rs:58-118) with the decoder as the model: the prompt is fed through the KV cache one position
 * at a time from position 0, then up to max_tokens tokens are sampled on the host from the logits of each decode
 * step.  generated_out holds max_tokens entries; *n_generated tells how many were produced (EOS stops early and is
 * not stored). */
int32_t yscv_hip_decoder_generate(yscv_hip_decoder *d, const uint32_t *input_ids, size_t n_input,
                                  const yscv_hip_generate_config *cfg, uint32_t *generated_out,
                                  size_t *n_generated);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* YSCV_HIP_H */
