/*
 * driss_torch_hip.h -- C ABI of the MI355X (gfx950) FP8 / MX quantization kernels.
 *
 * Plain pointers and sizes only: no torch types, no C++ types, no exceptions.  Every entry
 * point validates its arguments on the host, enqueues its kernels on `stream` (NULL = the
 * legacy default stream), never synchronises, never allocates device memory, and returns a
 * dt_status code.  (One exception to "never allocates", for callers that opted in with
 * dt_set_exclusive_gpu / DRISS_TORCH_RESIDENT only: the one-kernel path of the per-tensor dynamic
 * quantization keeps one 64-byte block of pinned HOST memory per device, made by dt_set_exclusive_gpu(1)
 * or at the first such launch, see dt_dynamic_scaled_quant.)  All data pointers are device pointers on
 * the current HIP device.
 *
 * Each declaration cites the reference (drisspg/driss_torch) interface it stands in for;
 * paths are relative to the reference tree.  The torch-facing registration shim
 * (driss_torch_amd/csrc/register_ops.cpp) keeps the TORCH_LIBRARY(DrissTorch) schemas of
 * src/register_ops.cpp:13-43 and calls only these functions.
 */
#ifndef DRISS_TORCH_HIP_H
#define DRISS_TORCH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DT_API __attribute__((visibility("default")))

/* hipStream_t without pulling in the HIP headers */
typedef struct ihipStream_t* dt_stream_t;

enum dt_status {
  DT_OK = 0,
  DT_ERR_INVALID_DTYPE = 1,   /* in/out dtype code not supported by this entry point */
  DT_ERR_INVALID_SHAPE = 2,   /* negative size, or a divisibility requirement not met */
  DT_ERR_NULL_POINTER = 3,
  DT_ERR_MISALIGNED = 4,      /* pointer alignment requirement not met */
  DT_ERR_WORKSPACE = 5,       /* workspace missing or too small */
  DT_ERR_INVALID_MODE = 6,    /* round_mode / axis / layout code out of range */
  DT_ERR_LAUNCH = 7,          /* hipGetLastError() after the launch was not hipSuccess */
  DT_ERR_EMPTY = 8,           /* reduction over zero elements */
  DT_ERR_RESIDENT_GAVE_UP = 9,/* an EARLIER per-tensor dynamic quantization on this device gave up waiting for
                                 the whole chip and wrote NaN outputs (see dt_dynamic_scaled_quant); nothing
                                 was launched by this call; the one-kernel path is off from now on */
  DT_ERR_TOO_LARGE = 10       /* more elements than dt_dynamic_scaled_quant_noalloc takes (DT_NOALLOC_MAX_NUMEL) */
};

/* element types of the high-precision operand */
enum dt_in_dtype { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };
/* OCP FP8 output types */
enum dt_out_dtype { DT_E4M3FN = 0, DT_E5M2 = 1 };

/*
 * How the product x*scale is rounded for a bf16 `x` before the fp8 convert (fp32 input:
 * the three coincide).  These are the three answers eager PyTorch gives for
 * test/test_sat_cast.py:7-24 depending on the scale tensor:
 *   DT_ROUND_BF16_PRODUCT        bf16(f32(x) * s)              0-dim CPU scale
 *   DT_ROUND_BF16_SCALE_PRODUCT  bf16(f32(x) * f32(bf16(s)))   0-dim device scale; what the
 *                                                              reference kernel computes,
 *                                                              src/saturated_cast.cu:66,81
 *   DT_ROUND_F32                 f32(x) * s                    scale of rank >= 1
 */
enum dt_round_mode { DT_ROUND_BF16_PRODUCT = 1, DT_ROUND_BF16_SCALE_PRODUCT = 2, DT_ROUND_F32 = 3 };

/* layout of the E8M0 scale bytes written by dt_mx_fp8_quantize */
enum dt_scale_layout {
  DT_SCALE_PLAIN = 0,   /* row-major [rows, blocks]: what src/mx_cast.cu:197-199,210-211 emits */
  DT_SCALE_BLOCKED = 1  /* 128x4 interleaved tiles: what src/mx_fp8_bf16.cu:197-205 consumes */
};

DT_API const char* dt_status_string(int status);
DT_API int dt_abi_version(void);

/* ------------------------------------------------------------------ workspace --------
 * dt_amax and dt_dynamic_scaled_quant combine per-workgroup partial maxima through a
 * small device workspace (partials + an arrival counter).  The caller owns it: allocate
 * dt_workspace_bytes() bytes (256-byte aligned), call dt_workspace_init once, then reuse
 * it for any number of calls that are ordered on one stream.  Calls that may overlap on
 * the device need separate workspaces.  (The reference allocates its scratch per call
 * from the torch allocator: src/amax.cu:115, src/dynamic_scaled_quant.cu:172.)          */
DT_API size_t dt_workspace_bytes(void);
DT_API int dt_workspace_init(void* workspace, size_t workspace_bytes, dt_stream_t stream);

/* ------------------------------------------------------------------ amax -------------
 * out[0] = max_i |x_i| as fp32 (NaN if any x_i is NaN).  Replaces driss_torch::amax,
 * src/amax.cu:106-119 (host) and :70-102 (kernel + launch).  x: DT_F32 or DT_BF16, any
 * numel >= 1 (the reference needs an even numel, src/amax.cu:113), any alignment of the
 * element type.                                                                          */
DT_API int dt_amax(const void* x, int in_dtype, int64_t numel, float* out, void* workspace,
                   size_t workspace_bytes, dt_stream_t stream);

/* ------------------------------------------------------------ saturated_cast ---------
 * out[i] = fp8_rne(clamp(x[i] * scale[0], -fmax, fmax)), NaN kept.  Replaces
 * driss_torch::saturated_cast, src/saturated_cast.cu:227-252 (host), :168-224 (dispatch),
 * :38-153 (kernels).  `scale` is one fp32 value in device memory.  The elements are taken
 * in storage order, so a column-major input gives a column-major output exactly as
 * src/saturated_cast.cu:243-249 does.  numel >= 0.                                       */
DT_API int dt_saturated_cast(const void* x, int in_dtype, int64_t numel, const float* scale,
                             int out_dtype, int round_mode, void* out, dt_stream_t stream);

/* -------------------------------------------------------- dynamic_scaled_quant -------
 * Per tensor: amax = max|x|, scale = f32(fmax / max(f64(amax), 1e-12)), out as
 * dt_saturated_cast.  Replaces driss_torch::dynamic_scaled_quant,
 * src/dynamic_scaled_quant.cu:157-176 (host), :119-153 (launch), :83-118 (kernel); the
 * scale formula is the one its test checks, test/test_dynamic_quant.py:36 (the kernel's
 * own `fmax / (amax + 1e-12)` at :111 differs in the last bits).  amax_out / scale_out may
 * be NULL.  The reference runs fp32 input only (:130,135); bf16 is accepted here.
 *
 * With the opt-in below, a tensor that fits the chip (128 MiB on 256 CUs, up to 4 x that partly) is quantized by ONE kernel
 * that occupies every CU and waits inside for all of its workgroups, where the reference uses a
 * cooperative launch (:144-150).  That assumes THIS PROCESS OWNS THE GPU: the library chains such
 * launches of one process, and avoids streams with a CU mask, processes with a CU mask in the
 * environment and streams under graph capture, but it cannot see another process.  If the chip is
 * not free within a bounded wait ("dynamic.resident_spin_limit"), the waiting workgroups give up:
 * their outputs, amax and scale are NaN, every kernel still runs to its end, a word of pinned host
 * memory is set, and the NEXT dt_dynamic_scaled_quant / _pair call on that device launches nothing,
 * returns DT_ERR_RESIDENT_GAVE_UP once and switches the one-kernel path off for the process
 * (calls after that take the two kernels).  The workspace stays
 * usable.  dt_dynamic_quant_gave_up() asks the same question without a quantization call: 1 if a
 * completed launch on the current device gave up since the last time it was asked (and clears it).
 *
 * Because of that assumption the one-kernel path is OFF unless the caller opts in: dt_set_exclusive_gpu(1)
 * (or DRISS_TORCH_RESIDENT=1 in the environment when the library is loaded; "0" or unset = off).  Without
 * the opt-in every call runs the reduction kernel followed by the cast kernel, which wait for nothing and
 * cannot produce NaN where the reference's cooperative launch could not.  dt_set_exclusive_gpu(1) also
 * makes the current device's block of pinned host memory, so that no later call allocates; with the
 * environment variable alone the first one-kernel launch on a device makes it.  The setting is one per
 * process, not per device, and so is the switch-off after a give-up.  dt_get_exclusive_gpu() returns it;
 * dt_dynamic_quant_resident_launches() counts the one-kernel launches of this process so far.
 * The call that returns DT_ERR_RESIDENT_GAVE_UP wrote nothing to its outputs: repeat it.             */
DT_API int dt_set_exclusive_gpu(int on);
DT_API int dt_get_exclusive_gpu(void);
DT_API uint64_t dt_dynamic_quant_resident_launches(void);
DT_API int dt_dynamic_quant_gave_up(void);
DT_API int dt_dynamic_scaled_quant(const void* x, int in_dtype, int64_t numel, int out_dtype,
                                   int round_mode, void* out, float* amax_out, float* scale_out,
                                   void* workspace, size_t workspace_bytes, dt_stream_t stream);

/* dt_dynamic_scaled_quant for callers that can neither allocate device memory nor keep a workspace
 * around: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference (whose op takes its scratch from the caching allocator on every
 * call, src/dynamic_scaled_quant.cu:172).  Same arguments and the same bits as
 * dt_dynamic_scaled_quant, without the workspace: the reduction's 4 KiB of scratch live in a device
 * array that is part of the library itself (one copy per GPU, held until the process ends).  The call
 * allocates and frees nothing -- no hipMalloc / hipFree, no pinned host memory -- and always runs as the
 * reduction kernel followed by the cast kernel (never the one-kernel path, which makes a block of host
 * memory at its first use and is refused under capture anyway); a small fill kernel clears the scratch's
 * counters first.  At most DT_NOALLOC_MAX_NUMEL elements, else DT_ERR_TOO_LARGE.  All calls on one GPU
 * share that GPU's array: calls that may overlap there (two streams, two threads) race on it and must
 * be ordered by the caller; use dt_dynamic_scaled_quant with a workspace per stream for those.  The
 * first call on a device looks the array's address up (hipGetSymbolAddress): make it outside a capture. */
#define DT_NOALLOC_MAX_NUMEL ((int64_t)1 << 34)
DT_API int dt_dynamic_scaled_quant_noalloc(const void* x, int in_dtype, int64_t numel, int out_dtype,
                                           int round_mode, void* out, float* amax_out, float* scale_out,
                                           dt_stream_t stream);

/* As above with two outputs from one read of x for the cast: e4m3fn with scale 448/amax and
 * e5m2 with scale 57344/amax.  scale_out, if given, receives {scale_e4m3fn, scale_e5m2}.
 * No counterpart in the reference (one dtype per call there).                             */
DT_API int dt_dynamic_scaled_quant_pair(const void* x, int in_dtype, int64_t numel, int round_mode,
                                        void* out_e4m3fn, void* out_e5m2, float* amax_out,
                                        float* scale_out, void* workspace, size_t workspace_bytes,
                                        dt_stream_t stream);

/* The two stages of dt_dynamic_scaled_quant_pair as separate calls, for callers that keep the
 * scales (delayed scaling: the reference's own flow is tensor_to_scale followed by
 * saturated_cast, test/test_sat_cast.py:35-38) or time the stages separately.
 * dt_amax_scales: amax_out[0] = max|x|, scale_out = {f32(448/max(amax,1e-12)),
 * f32(57344/max(amax,1e-12))}; either may be NULL, the scales are also left in the workspace.
 * dt_saturated_cast_pair: `scale` is that device pair; out_e4m3fn uses scale[0], out_e5m2
 * scale[1].                                                                               */
DT_API int dt_amax_scales(const void* x, int in_dtype, int64_t numel, float* amax_out, float* scale_out,
                          void* workspace, size_t workspace_bytes, dt_stream_t stream);
DT_API int dt_saturated_cast_pair(const void* x, int in_dtype, int64_t numel, const float* scale,
                                  int round_mode, void* out_e4m3fn, void* out_e5m2, dt_stream_t stream);

/* Row-wise: one amax / scale per row of a row-major [rows, cols] matrix, product in fp32
 * (a [rows,1] scale promotes in eager).  amax_out / scale_out: fp32 [rows] or NULL.  No
 * counterpart in the reference; the formulation is test/test_dynamic_quant.py:8-25 with
 * amax(dim=-1, keepdim=True).                                                             */
DT_API int dt_dynamic_scaled_quant_rowwise(const void* x, int in_dtype, int64_t rows, int64_t cols,
                                           int out_dtype, void* out, float* amax_out,
                                           float* scale_out, dt_stream_t stream);

/* -------------------------------------------------------------- mx_fp8_quantize ------
 * MXFP8 cast of a row-major [rows, cols] matrix: one E8M0 byte per 32 elements,
 * byte = clamp(ceil(log2(blockmax)) - P + 127, 0, 254) with P = 8 (e4m3fn) or 15 (e5m2),
 * payload = fp8_rne(clamp(x * 2^(127-byte))).  Replaces driss_torch::mx_fp8_quantize,
 * src/mx_cast.cu:168-246 (host), :96-161 (kernel), :44-86 (exponent math).
 *   axis 1: blocks along a row (the only mode of the reference); cols % 32 == 0
 *   axis 0: blocks down a column; rows % 32 == 0
 *   transpose 0: data [rows, cols]; scale [rows, cols/32] (axis 1) or [rows/32, cols] (axis 0)
 *   transpose 1: data [cols, rows]; scale [cols/32, rows] (axis 1) or [cols, rows/32] (axis 0)
 *                so (axis 0, transpose 1) equals the axis-1 cast of x^T.
 * scale_layout DT_SCALE_BLOCKED writes the scale matrix directly in the layout
 * dt_mx_fp8_bf16 reads (dt_blocked_scale_bytes(scale_rows, scale_cols) bytes, padding
 * zeroed); it needs the scale matrix to be [outer, inner/32], i.e. (axis 1, transpose 0)
 * or (axis 0, transpose 1).  in_dtype F32, BF16 or F16.  x only has to be aligned to its element (a
 * view that starts anywhere in its buffer keeps the 16-byte loads).  Shapes and output alignments the
 * tiled kernels do not take run on a much slower general kernel: data not 16-byte aligned (axis 1,
 * transpose 0: 8-byte), scale not 4-byte aligned (axis 0, transpose 0: 8-byte), cols not a multiple of
 * 4 for axis 0, rows not a multiple of 16 for (axis 1, transpose 1).                          */
DT_API int dt_mx_fp8_quantize(const void* x, int in_dtype, int64_t rows, int64_t cols, int axis,
                              int transpose, int out_dtype, int scale_layout, void* data,
                              uint8_t* scale, dt_stream_t stream);

/* Both blockings of one tensor from a single read: the (axis 1, transpose 0) result in
 * data_rows [rows, cols] / scale_rows [rows, cols/32] and the (axis 0, transpose 1) result in
 * data_cols_t [cols, rows] / scale_cols_t [cols, rows/32] -- x for a forward product and x^T
 * for the weight-gradient product.  Bit-identical to two dt_mx_fp8_quantize calls; rows % 32
 * == 0 and cols % 32 == 0.  scale_layout applies to both scale matrices.  No counterpart in
 * the reference, which has the row-wise cast only (src/mx_cast.cu:168-246).               */
DT_API int dt_mx_fp8_quantize_dual(const void* x, int in_dtype, int64_t rows, int64_t cols,
                                   int out_dtype, int scale_layout, void* data_rows,
                                   uint8_t* scale_rows, void* data_cols_t, uint8_t* scale_cols_t,
                                   dt_stream_t stream);

/* bytes of an [R, C] scale matrix in the blocked layout: 128*ceil(R/128) * 4*ceil(C/4) */
DT_API int64_t dt_blocked_scale_bytes(int64_t R, int64_t C);

/* plain [R, C] -> blocked (zero padded).  Stands in for transformer_nuggets' to_blocked,
 * which the reference's test applies between the cast and the GEMM, test/test_mx.py:31-32 */
DT_API int dt_to_blocked(const uint8_t* scale, int64_t R, int64_t C, uint8_t* out, dt_stream_t stream);

/* ------------------------------------------------------------------ mx_fp8_bf16 ------
 * out[M,N] (bf16, row stride ldo elements) = (A * 2^(sfa-127)) (B * 2^(sfb-127)), fp32
 * accumulation.  Replaces driss_torch::mx_fp8_bf16, src/mx_fp8_bf16.cu:217-241 (host),
 * :168-214 (operand contract), :36-163 (GEMM).  a: e4m3fn [M,K], row stride lda bytes;
 * b: the reference's [K,N] tensor with stride(0)==1, i.e. e4m3fn [N,K] with row stride ldb
 * bytes; sfa / sfb: E8M0 in the blocked layout, dt_blocked_scale_bytes(M, K/32) and
 * (N, K/32) bytes with the padding zero (dt_mx_fp8_quantize and dt_to_blocked write it so).  K % 32
 * == 0 (the reference's own checks leave K % 128 == 0 only: its expected scale length
 * 128 ceil(M/128) ceil(K/32), :197-205, equals the blocked layout's only then; here the length is
 * dt_blocked_scale_bytes and any whole number of MX blocks is taken; the K-blocks of the padding
 * count as zero).  lda % 16 == 0, ldb % 16 == 0, a, b 16-byte aligned
 * (:190-195), out 8-byte aligned, N % 4 == 0 and ldo % 4 == 0 (the reference asks N % 8, :187);
 * 256 rows of an operand must span less than 4 GiB (255*ld + K bytes); the operand itself
 * may be larger.                                                                         */
DT_API int dt_mx_fp8_bf16(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb,
                          int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out,
                          int64_t ldo, dt_stream_t stream);

/* ------------------------------------------------------------------ mx_fp4_bf16 ------
 * The same product with e2m1 operands.  Replaces driss_torch::mx_fp4_bf16,
 * src/mx_fp8_bf16.cu:243-271.  a: [M, K/2] bytes, b: [N, K/2] bytes (the reference's
 * [K/2, N] tensor with stride(0)==1), two e2m1 values per byte with the even element in
 * the low nibble; K counts elements, lda / ldb bytes.  Scales, alignment and shape
 * rules as for dt_mx_fp8_bf16 (K % 32 == 0).                                            */
DT_API int dt_mx_fp4_bf16(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb,
                          int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out,
                          int64_t ldo, dt_stream_t stream);

/* ------------------------------------------------------------------ mx_fp4_quantize --
 * MXFP4 operands for dt_mx_fp4_bf16: e2m1 pairs (first element of a pair in the low nibble) and one
 * E8M0 byte per 32 elements.  axis 1: blocks along the rows of x [rows, cols] -> payload
 * [rows, cols/2], scales [rows, cols/32]; axis 0: blocks down the columns, payload transposed ->
 * [cols, rows/2] (pairs of adjacent rows of x), scales [cols, rows/32], i.e. the axis-1 cast of x^T.
 * Scales plain (row-major) or blocked.  The reference has no such op: its GEMM test takes the
 * operands from torchao's MXTensor.to_mx(x, "fp4_e2m1", 32) (test/test_mx.py:17-21), whose default
 * scale is restated here: shared exponent floor(log2(max|x|)) - 2 from the fp32 exponent field,
 * clamped to [-127, 127]; payload = e2m1_rne_saturating(x * 2^-exponent).  A zero block gives byte
 * 0; a block that holds a NaN gives byte 255 and 0x7 in every nibble; an infinite maximum gives
 * byte 253.  The blocked dimension % 32 == 0.  axis 1: x 16-byte aligned, data 4-byte aligned,
 * rows * cols < 2^33; axis 0: cols % 4 == 0, x aligned to 4 elements, data 16-byte and scale
 * 4-byte aligned.                                                                          */
DT_API int dt_mx_fp4_quantize(const void* x, int in_dtype, int64_t rows, int64_t cols, int axis,
                              int scale_layout, void* data, uint8_t* scale, dt_stream_t stream);

/* ------------------------------------------------------------- mx_fp4_quantize_dual --
 * Both MXFP4 operands of x [rows, cols] from one read of it: the axis-1 cast (payload
 * [rows, cols/2], scales [rows, cols/32]) and the axis-0 cast (payload [cols, rows/2], scales
 * [cols, rows/32]), bit-identical to two calls of dt_mx_fp4_quantize.  No counterpart in the
 * reference (see dt_mx_fp4_quantize); the MXFP4 sibling of dt_mx_fp8_quantize_dual.
 * rows % 32 == 0 and cols % 32 == 0.  One kernel when data_rows is 4-byte, data_cols_t 16-byte and
 * both scale buffers 4-byte aligned and rows, cols < 2^31; otherwise the two single casts with
 * their own rules.                                                                            */
DT_API int dt_mx_fp4_quantize_dual(const void* x, int in_dtype, int64_t rows, int64_t cols,
                                   int scale_layout, void* data_rows, uint8_t* scale_rows,
                                   void* data_cols_t, uint8_t* scale_cols_t, dt_stream_t stream);

/* ------------------------------------------------- block-scaled GEMM with a workspace --
 * dt_mx_fp8_bf16 / dt_mx_fp4_bf16 (src/mx_fp8_bf16.cu:217-271; the reference takes its GEMM
 * workspace from the caching allocator at :148-151) with a caller-owned workspace of
 * dt_mx_gemm_workspace_bytes() bytes, 256-byte aligned.  With it a problem whose output tiles
 * leave most CUs idle (few rows or columns, long K) shares K between several workgroups per
 * tile; the result does not depend on their timing.  The first 1 KiB of the workspace must be
 * zero before the first call (dt_mx_gemm_workspace_init, or any memset) and is left zero by
 * every call; calls that may overlap on the device need workspaces of their own.
 * workspace == NULL behaves as the plain entry point.                                     */
DT_API size_t dt_mx_gemm_workspace_bytes(void);
DT_API int dt_mx_gemm_workspace_init(void* workspace, size_t workspace_bytes, dt_stream_t stream);
DT_API int dt_mx_fp8_bf16_ws(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb,
                             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out,
                             int64_t ldo, void* workspace, size_t workspace_bytes, dt_stream_t stream);
DT_API int dt_mx_fp4_bf16_ws(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb,
                             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out,
                             int64_t ldo, void* workspace, size_t workspace_bytes, dt_stream_t stream);

/* ---------------------------------------------------------------- tuning -------------
 * Launch-shape knobs for benchmarking sweeps ("amax.blocks_per_cu", ...).  Returns DT_OK
 * or DT_ERR_INVALID_MODE for an unknown key.  Not part of the reference's surface.        */
DT_API int dt_set_tuning(const char* key, int value);
DT_API int dt_get_tuning(const char* key, int* value);

#ifdef DT_PHASE_LOG
/* Benchmarking aid, no counterpart in the reference, and NOT part of the product library: it exists only
 * in a second build of the kernels with -DDT_PHASE_LOG (python driss_torch_amd/_build.py --phase-log ->
 * lib/libdriss_torch_hip_phases.so), which the benchmark loads for its per-phase report.  While a device
 * buffer is set here (8-byte aligned, at least 32 bytes per workgroup of the kernel's grid, 64 for the
 * GEMM; NULL switches it off), every one-kernel dynamic quantization, amax reduction and block-scaled GEMM
 * launched on the buffer's device writes readings of the 100 MHz constant-rate counter per workgroup into
 * it (uint64[workgroup][4]: start; share loaded and reduced / loaded; released from the grid barrier /
 * workgroup maximum known; stores done / atomics done).  The buffer must outlive every such launch;
 * launches on other devices ignore it.                                                              */
DT_API int dt_set_phase_log(void* device_buffer, size_t bytes);
#endif

#ifdef __cplusplus
}
#endif
#endif /* DRISS_TORCH_HIP_H */
