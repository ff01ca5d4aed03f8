/*
 * tpq.h - C ABI of the gfx950 (MI355X) quantized-linear kernel library.
 *
 * Conventions shared by every entry point:
 *   - all tensor arguments are raw DEVICE pointers owned by the caller; the
 *     library never allocates, frees or keeps them;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     work is enqueued on it and the call returns without synchronising;
 *   - the return value is 0 on success and a TPQ_ERR_* code otherwise; the
 *     text of the last failure on the calling thread is tpq_last_error();
 *   - zero-sized problems succeed without launching anything;
 *   - floating tensors carry a TPQ_DTYPE_* tag; 16-bit floats are raw bits.
 *
 * Each entry point names the operator of the TensorPlay reference it stands
 * behind (paths relative to the reference root).
 */
#ifndef TPQ_H
#define TPQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPQ_DTYPE_F32 0
#define TPQ_DTYPE_F16 1
#define TPQ_DTYPE_BF16 2

#define TPQ_OK 0
#define TPQ_ERR_INVALID_VALUE 1 /* reference raises ValueError  */
#define TPQ_ERR_INVALID_TYPE 2  /* reference raises TypeError   */
#define TPQ_ERR_RUNTIME 3       /* HIP launch / runtime failure */
#define TPQ_ERR_UNSUPPORTED 4   /* valid in the reference, not built here */

/* Library ABI version (bumped on any signature change). */
int tpq_abi_version(void);

/* Message of the most recent non-zero return on this thread ("" if none). */
const char* tpq_last_error(void);

/*
 * Which kernel serves a call is a function of the call's arguments alone; the library never reads the environment and
 * has no switch that changes a route.
 */

/*
 * Fused row-wise signed quantizer.
 *   absmax = max_k |x[m,k]|; scale = max(absmax, eps) / divisor;
 *   code = clamp(rint(x / scale), qmin, qmax)   (sign_mode: x >= 0 ? qmax : qmin)
 * Replaces _quantize_int8_rowwise (divisor 127, [-127,127]),
 * _quantize_int4_rowwise (7, [-8,7]), _quantize_int2_rowwise (2, [-2,1]) and
 * _quantize_binary_rowwise (1, sign mode):
 *   config/native_functions.yaml:5338-5347,
 *   p10/src/backend/cuda/QuantGemmKernels.cu:1421-1609,
 *   p10/src/backend/cuda/LowBitGemmKernels.cu:27-76.
 * x [M,K] contiguous of x_dtype; codes int8 [M,K]; scales f32 [M].
 */
int tpq_quantize_rowwise(const void* x, int x_dtype, int64_t M, int64_t K, float eps,
                         float divisor, int qmin, int qmax, int sign_mode, int8_t* codes,
                         float* scales, void* stream);

/*
 * Integer matrix product C[M,N] (int32) = A[M,K] (int8, or uint8 when
 * a_unsigned) x B[K,N] (int8).  B is addressed as b[k*b_stride_k + n*b_stride_n]
 * so both a contiguous [K,N] operand (N,1) and the transposed view of a
 * contiguous [N,K] weight (1,K) are accepted without a copy.
 * Replaces _int_mm / _int_mm.out: config/native_functions.yaml:7987-7989,
 * p10/src/backend/cuda/IntMM.cu:383-454.
 */
int tpq_int_mm(const void* a, int a_unsigned, const int8_t* b, int64_t b_stride_k,
               int64_t b_stride_n, int32_t* c, int64_t M, int64_t K, int64_t N, void* stream);

/*
 * out[m,n] (f32) = (float(acc[m,n]) * row_scale[m]) * col_scale[n].
 * Replaces _int8_mm_rescale: config/native_functions.yaml:5350,
 * p10/src/backend/cuda/QuantGemmKernels.cu:1611-1650.
 */
int tpq_int8_mm_rescale(const int32_t* acc, const float* row_scale, const float* col_scale,
                        float* out, int64_t M, int64_t N, void* stream);

/*
 * Fused int8 GEMM + dequant epilogue: out[m,n] = cast_out(
 *   (float(sum_k a[m,k]*w[n,k]) * row_scale[m]) * col_scale[n] (+ bias[n])).
 * a int8 [M,K], w int8 [N,K] (both K-contiguous), bias f32 [N] or NULL,
 * out [M,N] of out_dtype.  One launch for the pair _int_mm + _int8_mm_rescale
 * that _int8_mm issues (tensorplay/ao/quantization/int8_mixed_precision.py:60-77)
 * and, with bias, the add at :242.
 */
int tpq_int8_mm_dequant(const int8_t* a, const int8_t* w, const float* row_scale,
                        const float* col_scale, const float* bias, void* out, int out_dtype,
                        int64_t M, int64_t N, int64_t K, void* stream);

/*
 * The same operation with a caller-provided workspace (16-byte aligned).  With few output tiles and a long K
 * (a few hundred rows against a square weight) the k range is cut into slices, one workgroup each, whose exact
 * integer partial sums go to the workspace; a second kernel adds them and applies the scales.  The result is
 * bit-identical to tpq_int8_mm_dequant (same reference lines).  tpq_int8_mm_workspace_bytes says how many
 * bytes the shape can use (0: the workspace would not be used); a NULL or smaller workspace falls back to
 * tpq_int8_mm_dequant.
 */
int64_t tpq_int8_mm_workspace_bytes(int64_t M, int64_t N, int64_t K);
/* tpq_int_mm (same reference lines: p10/src/backend/cuda/IntMM.cu:344-454) with the same optional workspace. */
int tpq_int_mm_ws(const void* a, int a_unsigned, const int8_t* b, int64_t b_stride_k,
                  int64_t b_stride_n, int32_t* c, int64_t M, int64_t K, int64_t N,
                  void* workspace, int64_t workspace_bytes, void* stream);
int tpq_int8_mm_dequant_ws(const int8_t* a, const int8_t* w, const float* row_scale,
                           const float* col_scale, const float* bias, void* out, int out_dtype,
                           int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                           void* stream);

/*
 * tpq_int8_mm_dequant_ws without the workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  The slice matrices live in a buffer built into the library, tpq_int8_mm_noalloc_max_bytes()
 * (16 MiB) per GPU, held until the process ends; the call allocates and frees nothing.  A shape whose slices
 * need more (tpq_int8_mm_workspace_bytes(M, N, K) above the maximum, e.g. 512 x 4096 x 4096) is rejected with
 * TPQ_ERR_INVALID_VALUE and belongs to tpq_int8_mm_dequant_ws;
 * a shape that uses no workspace runs as tpq_int8_mm_dequant.  Same result bits as tpq_int8_mm_dequant(_ws).
 * All calls on one GPU share that GPU's buffer: calls that overlap in time on one GPU (two streams, two
 * threads) race; order them on one stream or with events.
 */
int64_t tpq_int8_mm_noalloc_max_bytes(void);
int tpq_int8_mm_dequant_noalloc(const int8_t* a, const int8_t* w, const float* row_scale,
                                const float* col_scale, const float* bias, void* out, int out_dtype,
                                int64_t M, int64_t N, int64_t K, void* stream);

/*
 * int32 codes [N,K] in 0..15 -> int32 [ceil(N/8)][ceil(K/(16 I))][32][I/2],
 * the packed layout of the reference's device op (I = inner_k_tiles in {2,4,8}).
 * Replaces _convert_weight_to_int4pack: config/native_functions.yaml:7991,
 * p10/src/backend/cuda/QuantGemmKernels.cu:322-330, 838-877, 1349-1408.
 */
int tpq_int4_pack(const int32_t* codes, int64_t N, int64_t K, int inner_k_tiles, int32_t* out,
                  void* stream);

/*
 * y[m,n] = sum_k x[m,k] * ((code[n,k] - 8) * scale[k/g,n] + zero[k/g,n]).
 * x [M,K] and y [M,N] of `dtype`; packed as written by tpq_int4_pack with
 * inner_k_tiles = 2 and N = 8 * (first packed dimension); scales_and_zeros
 * [ceil(K/g), N, 2] of `dtype`; g in {32,64,128}.
 * Replaces _weight_int4pack_mm: config/native_functions.yaml:7993,
 * p10/src/backend/cuda/QuantGemmKernels.cu:1210-1341.
 */
int tpq_int4_mm(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed,
                int inner_k_tiles, int64_t N, int64_t group, const void* scales_and_zeros,
                void* out, void* stream);

/*
 * Same operator with a caller-provided scratch buffer, which lets the decode
 * kernel slice the k range of a column group across several workgroups (all
 * compute units busy when N/64 is small against their number).
 *   workspace: device memory, 16-byte aligned, at least
 *              tpq_int4_mm_workspace_bytes(N) bytes, ZERO-FILLED once after
 *              allocation; every call leaves its first 16 KiB (the arrival
 *              counters) zero again, so the buffer can be reused call after
 *              call.  Calls that share a workspace must not overlap in time
 *              (one workspace per stream).  NULL or too small = the
 *              single-workgroup path of tpq_int4_mm.
 * Results do not depend on the slicing order (partials are added in slice
 * order), so repeated calls are bit-identical.
 */
size_t tpq_int4_mm_workspace_bytes(int64_t N);
/* The same for a call with M rows: 113 .. 256 rows run on the tiled kernel, which with few tiles deals the steps of K to
 * up to 16 slices and keeps their fp32 sums [slice][M][N] behind the counters; never less than
 * tpq_int4_mm_workspace_bytes(N).  With a smaller workspace the call takes fewer slices or none: same roundings of the
 * weights, the sums added in another order. */
size_t tpq_int4_mm_rows_workspace_bytes(int64_t M, int64_t N, int64_t K);
int tpq_int4_mm_ws(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed,
                   int inner_k_tiles, int64_t N, int64_t group, const void* scales_and_zeros,
                   void* out, void* workspace, size_t workspace_bytes, void* stream);

/*
 * int8 ternary codes [rows, cols] <-> uint8 [rows, ceil(cols/4)], four 2-bit
 * fields per byte, first code in the two most significant bits.
 * Replace pack_ternary / unpack_ternary:
 * tensorplay/ao/quantization/bitnet.py:72-107.
 */
int tpq_ternary_pack(const int8_t* codes, int64_t rows, int64_t cols, uint8_t* out, void* stream);
int tpq_ternary_unpack(const uint8_t* packed, int64_t rows, int64_t cols, int8_t* out,
                       void* stream);

/*
 * BitNet packed linear after the activation quantizer:
 *   acc[m,n] = sum_k x[m,k] * code[n,k]               (int32, exact)
 *   out[m,n] = cast((float(acc) * row_scale[m]) * w_scale (+ bias[n]))
 * x int8 [M,K]; packed uint8 [N, ceil(K/4)]; bias f32 [N] or NULL; acc_out
 * int32 [M,N] or NULL (for parity checks); out [M,N] of out_dtype or NULL.
 * Replaces the unpack + PackedWeight.run + rescale sequence of
 * bitnet_linear_packed: tensorplay/ao/quantization/bitnet.py:215-241.
 */
int tpq_ternary_mm(const int8_t* x, const float* row_scale, const uint8_t* packed, float w_scale,
                   const float* bias, int64_t M, int64_t N, int64_t K, void* out, int out_dtype,
                   int32_t* acc_out, void* stream);
/*
 * The same product (same reference lines) with an optional device workspace.  From 33 rows on with
 * K > 2560 the fastest kernel cuts K into splits whose exact int32 partial sums go to the workspace
 * ([splits][M][N]) and are added by a second kernel: bit-identical results.  tpq_ternary_mm_workspace_bytes
 * says how many bytes the shape can use (0: none needed); a NULL or smaller workspace runs
 * tpq_ternary_mm's kernels.  Nothing has to be cleared between calls.
 */
int64_t tpq_ternary_mm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int tpq_ternary_mm_ws(const int8_t* x, const float* row_scale, const uint8_t* packed, float w_scale,
                      const float* bias, int64_t M, int64_t N, int64_t K, void* out, int out_dtype,
                      int32_t* acc_out, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Two fusions around the decode matmul for the MLP of a decoder layer (float16 / bfloat16
 * activations, innerKTiles = 2, group 128, K % 128 == 0; anything else returns TPQ_ERR_UNSUPPORTED
 * and the caller runs the separate ops).  Both round exactly where the separate ops would.
 *   tpq_int4_mm_add:    out = T(T(x . W^T) + residual)            (residual, out: [M, N] of dtype)
 *   tpq_int4_mm_swiglu: out = silu_mul(T(x . Wgate^T), T(x . Wup^T)) = T(g * sigmoid(g) * u) in fp32
 * They stand for _weight_int4pack_mm followed by add, and for two _weight_int4pack_mm calls
 * followed by silu_mul (config/native_functions.yaml:6071-6075,
 * p10/src/backend/cpu/PointwiseKernels.cpp:1466-1540), the sequence of the reference's decoder layer
 * (benchmark/bench_llama_e2e.py:140-144).
 */
int tpq_int4_mm_add(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed,
                    int inner_k_tiles, int64_t N, int64_t group, const void* scales_and_zeros,
                    const void* residual, void* out, void* stream);
int tpq_int4_mm_swiglu(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed_gate,
                       const int32_t* packed_up, int inner_k_tiles, int64_t N, int64_t group,
                       const void* sz_gate, const void* sz_up, void* out, void* stream);

/*
 * `count` (1..4) int4 weights applied to the same activations in one launch per 16 rows (per 32 rows where the
 * kernel takes two blocks of 16 rows against the same weight registers: K = 3072..4096, one pass of workgroups):
 * out[w] = T(x . W[w]^T), out[w]: [M, N[w]] of dtype, for w < count.  Same kernel, same shapes
 * (float16 / bfloat16, innerKTiles = 2, group 128, K % 128 == 0, else TPQ_ERR_UNSUPPORTED) and same
 * result as `count` calls of tpq_int4_mm at up to 16 rows per call.  packed, N, scales_and_zeros and
 * out are host arrays of `count` entries (device pointers / widths).  It stands for the three
 * _weight_int4pack_mm calls on one input that compute q, k and v in the reference's decoder layer
 * (benchmark/bench_llama_e2e.py:128-130): at 4096 x 4096 a launch costs more than the transfer of
 * its weight, so one launch for the three takes about half the time of three.
 */
int tpq_int4_mm_multi(const void* x, int dtype, int64_t M, int64_t K, int count,
                      const int32_t* const* packed, int inner_k_tiles, const int64_t* N, int64_t group,
                      const void* const* scales_and_zeros, void* const* out, void* stream);

/*
 * The two entry points above with the RMS normalization of the activations in front, the norm -> projection
 * pairs of a decoder layer (benchmark/bench_llama_e2e.py:126-128 q, k, v after n1; :143 gate and up after n2):
 *   xn = rms_norm(x, norm_weight, eps) = T((float(x) * rsqrt(mean(float(x)^2) + eps)) * float(norm_weight)),
 * computed in fp32 and rounded once to the activation dtype (tensorplay/nn/functional.py:2350-2372; native op
 * rms_norm, config/native_functions.yaml:5962), then out = the product with xn as above.  norm_weight: [K] of
 * dtype.  The kernel takes the row factor rsqrt(mean + eps) out of the sum: it multiplies T(x * norm_weight) with
 * the weights and scales the finished fp32 sums of a row, so no launch and no round trip of the activations through
 * memory is spent on the norm; the result differs from the two-step formulation only in where the rounding to T
 * falls and agrees with it to the tolerance of the product (1e-2 relative; 1e-3 against exact sums for float16).
 * Input range: any finite x and norm_weight of the dtype.  For float16 the product x * norm_weight can leave the
 * type's range (beyond 65504, or below 6e-5 where it loses its mantissa) although the normalized value does not, so
 * there every wavefront first scales both factors by exact powers of two taken from its own part of the row (the
 * scaled products stay within [-4, 4]) and multiplies its fp32 partial sums by the inverse power before they are
 * added; rows of magnitude 1e-4 .. 1e4 with weights 0.02 .. 30 hold the tolerance row by row.  bfloat16 has
 * float32's exponent range and needs none of it.
 * Built for K = 2048..8192 (the pair: 2049..4096) at up to 16 rows (the pair: 8); other shapes return
 * TPQ_ERR_UNSUPPORTED and the caller runs the norm and the plain entry point.
 */
int tpq_int4_mm_swiglu_norm(const void* x, int dtype, int64_t M, int64_t K, const void* norm_weight, float eps,
                            const int32_t* packed_gate, const int32_t* packed_up, int inner_k_tiles,
                            int64_t N, int64_t group, const void* sz_gate, const void* sz_up, void* out,
                            void* stream);
int tpq_int4_mm_multi_norm(const void* x, int dtype, int64_t M, int64_t K, const void* norm_weight, float eps,
                           int count, const int32_t* const* packed, int inner_k_tiles, const int64_t* N,
                           int64_t group, const void* const* scales_and_zeros, void* const* out, void* stream);

/*
 * rms_norm over the last dimension (native op rms_norm, config/native_functions.yaml:5962; CPU kernel
 * p10/src/backend/cpu/NormalizationKernels.cpp:1355-1453; Python composite tensorplay/nn/functional.py:2350-2372):
 *   out[m][k] = T((float(x[m][k]) * inv[m]) * float(weight[k])),  inv[m] = 1 / sqrt(mean_k(float(x[m][k])^2) + eps),
 * all in fp32, one rounding to `dtype` (float32 / float16 / bfloat16).  x, out: [M, K] contiguous; weight: [K] of
 * `dtype` or null (no scaling).  The sum of squares is added in a tree order, the reference's CPU kernel adds serially:
 * results agree to an ulp of `dtype`, not bit for bit.  It is the stand-alone form of the norm that
 * tpq_int4_mm_multi_norm / tpq_int4_mm_swiglu_norm fold into the matmul at decode sizes.
 */
int tpq_rms_norm(const void* x, int dtype, int64_t M, int64_t K, const void* weight, float eps, void* out,
                 void* stream);

/*
 * The linear, float-output form of _quantized_packed_run with the weight prepacked by _quantized_weight_prepack
 * (config/native_functions.yaml:11883-11886; CPU kernels
 * p10/src/backend/cpu/QuantPacked.cpp:420-516 and :519-572, packed_real_value p10/include/QuantPacked.h:133-139):
 *   acc[m][n] = sum_k x[m][k] w[n][k] - x_zero_point offsets[n] - w_zero_points[n] sum_k x[m][k]
 *               + K x_zero_point w_zero_points[n]                                   (integers, exact)
 *   out[m][n] = fmaf(float(acc), float(x_scale) * w_scales[n], bias ? bias[n] : 0);  relu: max(out, 0)
 * x: [M, K] int8 or uint8 codes of a per-tensor quantized activation; packed: [N, packed_row_stride] int8 with
 * packed_row_stride >= K (the reference pads rows to a multiple of 32 with zeros); offsets[n] = sum_k w[n][k] (int64),
 * w_scales [N] float32, w_zero_points [N] int64, bias [N] float32 or null; out: [M, N] float32.  K <= 65536.
 * workspace: device memory, 16-byte aligned, tpq_packed_linear_workspace_bytes(M, N, K, x_unsigned) bytes (the int32
 * products, and a signed copy of unsigned activations); contents need not be preserved between calls.
 * Bit-exact with the reference's arithmetic.  The convolution, requantised-output and activation forms are not built.
 */
size_t tpq_packed_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int x_unsigned);
int tpq_packed_linear_float(const void* x, int x_unsigned, double x_scale, int64_t x_zero_point, const int8_t* packed,
                            int64_t packed_row_stride, const int64_t* offsets, const float* w_scales,
                            const int64_t* w_zero_points, const float* bias, int relu, float* out, int64_t M, int64_t N,
                            int64_t K, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The plain GEMM of the reference's many-row route for packed weights, which dequantises the weight to a dense
 * matrix of the activation type and multiplies once (p10/src/backend/cuda/QuantGemmKernels.cu:1296-1341, the call
 * gemm_impl(xf, wf.t(), out, 1.0, 0.0, nullptr) at :1339; likewise behind _weight_int8pack_mm and the low-bit linear):
 *   out[m][n] = T(sum_k float(x[m][k]) * float(w[n][k])),  float32 accumulation, one rounding to `dtype`.
 * x: [M, K], w: [N, K] (the dense weight that tpq_int4_dequantize / tpq_int8pack_dequantize / tpq_lowbit_dequantize
 * wrote), out: [M, N], all contiguous and of `dtype` = float16, bfloat16 or float32; x and w 16-byte aligned.
 * TPQ_ERR_UNSUPPORTED for other types or K not a multiple of 64 (float32: of 32); nothing written then.
 */
int tpq_dense_mm(const void* x, int dtype, int64_t M, int64_t K, const void* w, int64_t N, void* out, void* stream);

/*
 * Dense weight [N, K] of `dtype` from the packed device layout: W = T(code - 8) * scale + zero, the
 * product and the sum each rounded to T.  The reference runs this before its library GEMM
 * (int4_tc_dequantize_kernel, p10/src/backend/cuda/QuantGemmKernels.cu:1170-1202, 1296-1341); the
 * host op uses it the same way for many activation rows.
 */
int tpq_int4_dequantize(const int32_t* packed, int inner_k_tiles, int64_t N, int64_t K, int64_t group,
                        const void* scales_and_zeros, int dtype, void* out, void* stream);

/*
 * int4 CPU layout written on the device: uint8 [N, K/2] as produced by the reference's CPU pack
 * (block_cols = 64 with half_split = 1 is the AVX-512 tier, 32/1 AVX2, 32/0 the plain tier).
 * Replaces _convert_weight_to_int4pack_for_cpu: config/native_functions.yaml:7997,
 * p10/src/backend/cpu/QuantizedElementwiseKernels.cpp:19, 370-390.
 */
int tpq_int4_pack_cpu_layout(const int32_t* codes, int64_t N, int64_t K, int block_cols,
                             int half_split, uint8_t* out, void* stream);

/*
 * CPU layout -> device layout (int32 [N/8][ceil(K/32)][32][1], innerKTiles = 2), so that a weight
 * packed by a CPU model (buffer `weight` of WeightOnlyInt4Linear,
 * tensorplay/ao/quantization/int4_weight_only.py:150-154) can be used by tpq_int4_mm.  The reference
 * has no such converter: its device op rejects the 2-D uint8 layout
 * (p10/src/backend/cuda/QuantGemmKernels.cu:1216-1254).
 */
int tpq_int4_cpu_layout_to_device(const uint8_t* packed_cpu, int64_t N, int64_t K, int block_cols,
                                  int half_split, int32_t* out, void* stream);

/*
 * int8 weight-only matmul: out[m,n] = cast((sum_k float(x[m,k]) * w[n,k]) * scales[n]), fp32
 * accumulation, out dtype = x dtype.  x [M,K] f32/f16/bf16; w int8 [N,K] row-major; scales f32 [N].
 * Replaces _weight_int8pack_mm: config/native_functions.yaml:8005,
 * p10/src/backend/cuda/QuantGemmKernels.cu:86-180, 339-405.
 */
int tpq_weight_int8pack_mm(const void* x, int dtype, int64_t M, int64_t K, const int8_t* w,
                           const float* scales, int64_t N, void* out, void* stream);

/*
 * Dense [N, K] weight of `dtype` from the int8 weight and its per-row scales: T(float(w) * scale[n]).
 * For many activation rows the host op multiplies this with tpq_dense_mm instead of streaming the
 * int8 weight once per 16 or 32 rows (the reference's device op runs its batched GEMV at every size,
 * p10/src/backend/cuda/QuantGemmKernels.cu:345-405).
 */
int tpq_int8pack_dequantize(const int8_t* w, const float* scales, int64_t N, int64_t K, int dtype,
                            void* out, void* stream);

/* Storage of quantized codes: one element per int8 / uint8 / int32, or 2 / 4 / 8 elements per byte
 * (element i in bits (i % pack) * bits of byte i / pack, i = row-major linear index). */
#define TPQ_STORAGE_I8 0   /* reference dtype qint8   */
#define TPQ_STORAGE_U8 1   /* quint8   */
#define TPQ_STORAGE_I32 2  /* qint32   */
#define TPQ_STORAGE_U4X2 3 /* quint4x2 */
#define TPQ_STORAGE_U2X4 4 /* quint2x4 */
#define TPQ_STORAGE_U1X8 5 /* quint1x8 */

/*
 * Block-wise affine quantizer: code = clamp(rint(x * (1 / scale[b])) + zero_point[b], quant_min,
 * quant_max), b = block of the element in the row-major grid of ceil(size / block_size) blocks
 * (block_size[d] >= sizes[d]: one block along d; 1: per index; else groups).  scale 0 acts as 1.
 * quant_min >= quant_max selects the storage's full range.
 * x: contiguous tensor of x_dtype with `ndim` (<= 8) dimensions; `sizes` and `block_size` are HOST
 * arrays; scales / zero_points are DEVICE f32 arrays with one entry per block or a single entry
 * (n_zeros = 0: no zero point); out: ceil(numel * bits / 8) bytes of `storage`.
 * Replaces quantize_affine: config/native_functions.yaml:5308-5312,
 * p10/src/backend/cpu/QuantKernels.cpp:365-455, 579-774,
 * p10/src/backend/cuda/AffineQuantKernels.cu:806-901.
 */
int tpq_quantize_affine(const void* x, int x_dtype, int ndim, const int64_t* sizes,
                        const int64_t* block_size, const float* scales, int64_t n_scales,
                        const float* zero_points, int64_t n_zeros, int storage, int64_t quant_min,
                        int64_t quant_max, void* out, void* stream);

/*
 * Inverse map: out (f32, shape `sizes`) = (float(code) - zero_point[b]) * scale[b].
 * Replaces dequantize_affine: config/native_functions.yaml:5314-5318,
 * p10/src/backend/cpu/QuantKernels.cpp:391-404, 440-455, 776-990.
 */
int tpq_dequantize_affine(const void* codes, int storage, int ndim, const int64_t* sizes,
                          const int64_t* block_size, const float* scales, int64_t n_scales,
                          const float* zero_points, int64_t n_zeros, float* out, void* stream);

/*
 * Weight-only matmul on packed n-bit weights (1 <= bits <= 8):
 *   out[m,n] = sum_k x[m,k] * (code[n,k] - zero[g,n]) * scale[g,n] (+ bias[n]),  g = k / group.
 * packed: uint8 [N, ceil(K / (8 / bits))]; code i of a byte sits in bits 8 - (i+1) * bits .. when
 * lsb_first = 0 (pack_intx / pack_int2) and in bits i * bits .. when lsb_first = 1 (pack_binary).
 * scales_and_zeros: f32 [K / group][N][2]; bias: f32 [N] or NULL; x, out: [M,K], [M,N] of `dtype`.
 * Replaces _intx_mm / _int2_mm / _binary_mm, which unpack, dequantize and call a float GEMM:
 * tensorplay/ao/quantization/intx_weight_only.py:35-133, int2_weight_only.py:63-139,
 * binary.py:50-95 (binary: scale' = 2 * scale, zero = 0.5, one group).
 */
int tpq_lowbit_mm(const void* x, int dtype, int64_t M, int64_t K, const uint8_t* packed, int bits,
                  int lsb_first, int64_t N, int64_t group, const float* scales_and_zeros,
                  const float* bias, void* out, void* stream);

/*
 * Dense [N, K] weight of `dtype` from the same packed form: (float(code) - zero) * scale
 * (_dequantize_intx, tensorplay/ao/quantization/intx_weight_only.py:110-124).
 */
int tpq_lowbit_dequantize(const uint8_t* packed, int bits, int lsb_first, int64_t N, int64_t K,
                          int64_t group, const float* scales_and_zeros, int dtype, void* out,
                          void* stream);

/*
 * codes uint8 [rows, cols] (values < 2^bits) <-> packed uint8 [rows, ceil(cols / (8 / bits))], the
 * last byte of a row padded with zero fields.  Replaces pack_intx / unpack_intx
 * (tensorplay/ao/quantization/intx_weight_only.py:35-80), pack_int2 / unpack_int2
 * (int2_weight_only.py:63-103) and, with lsb_first = 1, pack_binary / unpack_binary (binary.py:50-85).
 */
int tpq_lowbit_pack(const uint8_t* codes, int bits, int lsb_first, int64_t rows, int64_t cols,
                    uint8_t* packed, void* stream);
int tpq_lowbit_unpack(const uint8_t* packed, int bits, int lsb_first, int64_t rows, int64_t cols,
                      uint8_t* codes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TPQ_H */
