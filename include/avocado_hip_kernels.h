/*
 * avocado_hip_kernels.h
 *
 * The thin C-ABI layer between the host code of the backend (descriptors, validation, dispatch) and the
 * hand-written HIP kernels for gfx950.  Plain device pointers, sizes and a stream; nothing here knows
 * about descriptors.  Each launcher enqueues on `stream` and returns without synchronising.
 *
 * Return value of every launcher:
 *    0   launched (launch errors are picked up with hipGetLastError by the caller's status mapping)
 *   >0   a hipError_t
 *   AVHIP_NOT_SUPPORTED / AVHIP_UNSUPPORTED_DATATYPE / AVHIP_BAD_PARAM (negative)
 *
 * Data types are the integer values of avDataType_t.  Tensors are NHWC, weights [K, R, S, C], Winograd
 * matrices [t*t, tiles, C] with t = m + r - 1 and tile = (n*ceil(H/m) + th)*ceil(W/m) + tw
 * (src/activations.cuh:30-121 of the reference).  Scalars are passed as double and narrowed to the compute
 * type of the kernel (fp32 for fp16/bf16/fp32/int8 tensors, fp64 for fp64 tensors).
 */
#ifndef AVOCADO_HIP_KERNELS_H_
#define AVOCADO_HIP_KERNELS_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

#ifndef AVHIP_API
#  define AVHIP_API __attribute__((visibility("default")))
#endif

#define AVHIP_NOT_SUPPORTED (-1)
#define AVHIP_UNSUPPORTED_DATATYPE (-2)
#define AVHIP_BAD_PARAM (-3)

	/* Geometry of one 2-D convolution.  pad_* are Avocado's signed input offsets (3x3 "same" is -1). */
	typedef struct
	{
		int N, H, W, C; /* input  [N, H, W, C]  */
		int K, R, S; /* weights [K, R, S, C] */
		int Ho, Wo; /* output [N, Ho, Wo, K] */
		int pad_h, pad_w;
		int stride_h, stride_w;
		int dil_h, dil_w;
		int mode; /* avConvolutionMode_t */
	} avhipConvShape;

	/* U = G g G^T.  Replaces launch_weight_transform / kernel_winograd_weight_transform,
	 * src/winograd_nonfused.cu:609,257.  w dtype `dtype`, U dtype `mat_dtype`. */
	AVHIP_API int avhip_winograd_weight_transform(void *stream, int dtype, int mat_dtype, int m, int r, int invert, const void *w, void *U, int K, int C);

	/* V = B^T d B with offset padding.  Replaces launch_input_transform / kernel_winograd_input_transform,
	 * src/winograd_nonfused.cu:654,303.  padding_value points to a host scalar of type `dtype` or is null (0). */
	AVHIP_API int avhip_winograd_input_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *x, void *V, int N, int H, int W, int C,
			int pad_h, int pad_w, const void *padding_value);

	/* y = act(alpha1 * A^T M A + bias + alpha2 * z) + beta * y.  Replaces launch_output_transform /
	 * kernel_winograd_output_transform, src/winograd_nonfused.cu:704,367.  bias is fp32 (fp64 for fp64 tensors)
	 * or null, z has the dtype of y or is null. */
	AVHIP_API int avhip_winograd_output_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *M, void *y, const void *bias, const void *z,
			int N, int H, int W, int K, double alpha1, double alpha2, double beta, int activation);

	/* M = G' dy G'^T over non-overlapping m x m tiles of dy [N, H, W, K] (zeros past the border), M [t*t, tiles, K].
	 * Replaces launch_gradient_transform / kernel_winograd_gradient_transform, src/winograd_nonfused.cu:780,425. */
	AVHIP_API int avhip_winograd_gradient_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *dy, void *M, int N, int H, int W,
			int K);

	/* dw [K, r, r, C] = alpha * U' M U'^T + beta * dw, M [t*t, K, C].  Replaces launch_update_transform /
	 * kernel_winograd_update_transform, src/winograd_nonfused.cu:828,475. */
	AVHIP_API int avhip_winograd_update_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *M, void *dw, int K, int C, double alpha,
			double beta);

	/* C[b] = alpha * op(A[b]) op(B[b]) + beta * C[b], row-major.  Replaces the cuBLAS calls of cudaGemm and
	 * cudaGemmBatched, src/gemm.cpp:25-124,126-209.  ab_dtype: FLOAT16 / BFLOAT16 / FLOAT32 / FLOAT64 / INT8;
	 * c_dtype: same as ab_dtype, FLOAT32 for 16-bit inputs, INT32 for INT8.  Strides are in elements. */
	AVHIP_API int avhip_gemm_batched(void *stream, int ab_dtype, int c_dtype, int opA, int opB, const void *A, const void *B, void *C, int batch, int M, int N,
			int K, int lda, int ldb, int ldc, int64_t strideA, int64_t strideB, int64_t strideC, double alpha, double beta);

	/* y = act(alpha1 * conv(x, w) + bias + alpha2 * z) + beta * y by implicit GEMM on MFMA.  Replaces
	 * cuda_convolution2dImplicitGemm / kernel_conv_implicit_gemm, src/conv2d_implicit_gemm.cu:303,152.
	 *   x_dtype FLOAT16 / BFLOAT16 / FLOAT32 : y and z have x_dtype, bias is fp32
	 *   x_dtype INT8, y_dtype INT32, bias_dtype INT32, alpha1 == 1, beta == 0, no z, LINEAR or RELU: exact integers
	 *   x_dtype INT8 otherwise: fp32 epilogue on the int32 sum, bias fp32, y INT32 / INT8 / FLOAT32
	 *   requant_scale != null (x INT8, y INT8, bias INT32): y = sat_i8(rne(float(sum + bias) * scale[k]))
	 * padding_value points to a host scalar of x_dtype or is null (0). */
	AVHIP_API int avhip_conv2d_implicit_gemm(void *stream, int x_dtype, int y_dtype, int bias_dtype, const avhipConvShape *shape, const void *x, const void *w,
			const void *bias, const void *z, void *y, const void *padding_value, double alpha1, double alpha2, double beta, int activation,
			const float *requant_scale);

	/* Same formula by a single fused Winograd F(2x2, 3x3) kernel (3x3, stride 1, dilation 1).  Replaces
	 * cuda_winogradFusedForward / kernel_winograd_fused, src/winograd_fused.cu:789,590.
	 * U is the transformed weight set [16, K, C] in FLOAT16 (16-bit tensors) or FLOAT32 (fp32 tensors). */
	AVHIP_API int avhip_conv2d_winograd_fused(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias, const void *z,
			void *y, double alpha1, double alpha2, double beta, int activation);

	/* The same formula for 16-bit tensors by Winograd F(2,3) along image rows only, in one kernel (3x3, stride 1, dilation 1,
	 * zero padding value, C = 64, 128 or 256, K a multiple of 128, beta = 0, LINEAR or RELU, values inside the fp16 range;
	 * AVHIP_NOT_SUPPORTED for other layers, with nothing launched).  The four planes of the transformed domain stay in accumulator registers for the whole k loop, so
	 * the matrix cores do two thirds of the direct kernel's work and the output transform is paid once per output.  Stands
	 * where the reference has its fused prototype, cuda_winogradFusedForward, src/winograd_fused.cu:789 (which transforms in
	 * both directions).  U is what avhip_winograd_rows_weight_transform wrote: avhip_winograd_rows_weight_bytes(K, C) bytes
	 * of fp16 in the register layout of the kernel's MFMA operand, [C / 32][3][4][K / 32][2][64 lanes][8]. */
	AVHIP_API int avhip_conv2d_winograd_rows(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias, const void *z,
			void *y, double alpha1, double alpha2, double beta, int activation);
	/* U_p[i] = sum_j G[p][j] * w[k, i, j] for the kernel above (taps reversed when `invert`), w of `dtype` (FLOAT16 / BFLOAT16).
	 * Stands where the reference has kernel_winograd_weight_transform, src/winograd_nonfused.cu:257. */
	AVHIP_API int avhip_winograd_rows_weight_transform(void *stream, int dtype, int invert, const void *w, void *U, int K, int C);
	AVHIP_API int64_t avhip_winograd_rows_weight_bytes(int K, int C);
	/* Whether avhip_conv2d_winograd_rows takes the layer (0) or not (AVHIP_NOT_SUPPORTED), the number of workgroups it would
	 * launch and how many of a workgroup's 128 GEMM rows are output pixels pairs of the image: what a dispatcher weighs. */
	AVHIP_API int avhip_conv2d_winograd_rows_plan(int dtype, const avhipConvShape *shape, int *workgroups, int *rows_used);
	/* Tuning knob without a counterpart in the reference: 0 makes the plan above decline every layer (the dispatcher then uses
	 * the direct kernels), 1 (default) lets the dispatcher weigh it, 2 makes the dispatcher take it for every layer it can run
	 * (tests); a negative value changes nothing.  Returns the previous value. */
	AVHIP_API int avhip_set_winograd_rows(int mode);

	/* The same formula for 3x3 stride-2 layers of 16-bit tensors (dilation 1, zero padding value, C a multiple of 64, K a multiple of
	 * 256, beta = 0, LINEAR or RELU; AVHIP_NOT_SUPPORTED otherwise, with nothing launched): the input under a tile of output pixels
	 * lies in LDS as four parity planes, so that a filter tap is a constant shift of consecutive plane pixels, and the filters come
	 * straight from L2 in MFMA register layout.  Stands where the reference has cuda_convolution2dImplicitGemm,
	 * src/conv2d_implicit_gemm.cu:303 (stride 1 only there).  U is what avhip_conv2d_strided_weight_layout wrote:
	 * avhip_conv2d_strided_weight_bytes(K, C) bytes, the weights themselves in the order [C / 32][9][K / 32][2][64 lanes][8]. */
	AVHIP_API int avhip_conv2d_strided(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias, const void *z,
			void *y, double alpha1, double alpha2, double beta, int activation);
	AVHIP_API int avhip_conv2d_strided_weight_layout(void *stream, int dtype, int invert, const void *w, void *U, int K, int C);
	AVHIP_API int64_t avhip_conv2d_strided_weight_bytes(int K, int C);
	/* Whether avhip_conv2d_strided takes the layer (0) or not (AVHIP_NOT_SUPPORTED), its workgroups and the output pixels per
	 * workgroup (of 224 GEMM rows); avhip_set_conv_strided: 0 declines everything, 1 (default) lets the dispatcher weigh it, 2 makes
	 * the dispatcher take every layer it can run, negative changes nothing; returns the previous value. */
	AVHIP_API int avhip_conv2d_strided_plan(int dtype, const avhipConvShape *shape, int *workgroups, int *rows_used);
	AVHIP_API int avhip_set_conv_strided(int mode);

	/* 1x1 stride-1 convolution without padding of fp16 / bf16 tensors with C = 128 or 256 and a multiple of 512 filters, beta = 0,
	 * LINEAR or RELU: blocks of up to 224 pixels resident in LDS, filters from L2 in MFMA operand layout, results stored from the
	 * accumulators without a pass through LDS (csrc/conv_pointwise_block.hip).  Same arithmetic as the reference's implicit GEMM,
	 * src/conv2d_implicit_gemm.cu:303, for a 1x1 filter.  U is what avhip_conv2d_pointwise_block_weight_layout wrote:
	 * avhip_conv2d_pointwise_block_weight_bytes(K, C) bytes, the weights themselves in the order [K / 32][C / 16][64 lanes][8]. */
	AVHIP_API int avhip_conv2d_pointwise_block(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias,
			const void *z, void *y, double alpha1, double alpha2, double beta, int activation);
	AVHIP_API int avhip_conv2d_pointwise_block_weight_layout(void *stream, int dtype, const void *w, void *U, int K, int C);
	AVHIP_API int64_t avhip_conv2d_pointwise_block_weight_bytes(int K, int C);
	/* Whether avhip_conv2d_pointwise_block takes the layer (0) or not (AVHIP_NOT_SUPPORTED), its workgroups and the pixels per
	 * workgroup (of 224 GEMM rows); avhip_set_pointwise_block: 0 declines everything, 1 (default) lets the dispatcher weigh it, 2
	 * makes the dispatcher take it wherever it can run; a negative mode only reads.  Returns the previous mode. */
	AVHIP_API int avhip_conv2d_pointwise_block_plan(int dtype, const avhipConvShape *shape, int *workgroups, int *rows_used);
	AVHIP_API int avhip_set_pointwise_block(int mode);

	/* y = alpha1 * act(alpha2 * x + b + beta1 * z) + beta2 * z + beta3 * y.  Replaces kernel_add_bias,
	 * src/tensor_op.cu:199-228.  x, y, z have `dtype`; b is fp32 (fp64 for fp64 tensors). */
	AVHIP_API int avhip_add_bias(void *stream, int dtype, const void *x, const void *b, const void *z, void *y, int64_t first, int last, double alpha1,
			double alpha2, double beta1, double beta2, double beta3, int activation);

	/* Explicit im2row; strides and dilations of `shape` are honoured (the reference's kernel is stride 1 only).  Replaces
	 * kernel_im2row_conv2d, src/im2row.cu:29-66.  elem_size in bytes. */
	AVHIP_API int avhip_im2row(void *stream, int elem_size, const avhipConvShape *shape, const void *x, void *rows, const void *padding_value);

	/* y = alpha * act(x * weight[j] + bias[j]) + beta * y over a [first, last] view of x (j = last index).  Replaces
	 * kernel_affine_forward, src/batchnorm.cu:28-48.  weight, bias: fp32 (fp64 for fp64 tensors). */
	AVHIP_API int avhip_affine_forward(void *stream, int dtype, const void *x, void *y, const void *weight, const void *bias, int64_t first, int64_t last,
			double alpha, double beta, int activation);

	/* Batch normalisation in inference: the affine transform above with weight = scale / sqrt(variance + epsilon) and
	 * bias = bias - mean * weight, computed on the fly.  Replaces kernel_batchnorm_forward, src/batchnorm.cu:51-69. */
	AVHIP_API int avhip_batchnorm_inference(void *stream, int dtype, const void *x, void *y, const void *scale, const void *bias, const void *mean,
			const void *variance, int64_t first, int64_t last, double alpha, double beta, double epsilon, int activation);

	/* Element type conversion with round-to-nearest-even and saturation.  Replaces cudaChangeType's kernels,
	 * src/conversions.cu:253-258. */
	AVHIP_API int avhip_change_type(void *stream, void *dst, int dst_dtype, const void *src, int src_dtype, int64_t elements);

	/* Fills `bytes` bytes at dst with a repeating pattern of 1, 2, 4, 8 or 16 bytes.  Replaces kernel_setall,
	 * src/descriptors.cu:22-39. */
	AVHIP_API int avhip_set_memory(void *stream, void *dst, int64_t bytes, const void *pattern, int pattern_size);

	/* The implicit-GEMM forward with k split across workgroups, for layers with few output pixels and a long k (fewer than 256
	 * tiles of 128 x 128 and a walk that is worth cutting, by the launcher's estimate): parts of the k range are summed in
	 * fp32 into `workspace` ([parts][N * Ho * Wo][K] floats), a second kernel adds the parts and applies the same epilogue as
	 * avhip_conv2d_implicit_gemm (any activation).  fp32 / fp16 / bf16 tensors, y of the type of x, fp32 bias.  Returns
	 * AVHIP_NOT_SUPPORTED, with nothing launched, when the layer is not worth splitting, the workspace is smaller than
	 * avhip_conv2d_split_k_workspace() reports, or the tensors are not aligned for the branch-free loaders (the caller then
	 * uses avhip_conv2d_implicit_gemm).  No counterpart in the reference, whose prototype has one tiling
	 * (src/conv2d_implicit_gemm.cu:303-352). */
	AVHIP_API int avhip_conv2d_implicit_gemm_split_k(void *stream, int x_dtype, const avhipConvShape *shape, const void *x, const void *w, const void *bias,
			const void *z, void *y, const void *padding_value, double alpha1, double alpha2, double beta, int activation, void *workspace,
			int64_t workspace_bytes);
	/* Bytes of workspace with which avhip_conv2d_implicit_gemm_split_k takes the layer; 0 when it would not. */
	AVHIP_API int avhip_conv2d_split_k_workspace(int x_dtype, const avhipConvShape *shape, int64_t *bytes);

	/* Tuning knob without a counterpart in the reference.  The implicit-GEMM launcher sends a convolution to the kernel with
	 * one 32 x 32 tile per wavefront when its 128 x 128 tiling would yield fewer than this many workgroups (default 192 on
	 * the 256 compute units of an MI355X) and its k extent is short enough for that kernel to be the faster one by the
	 * launcher's estimate; 0 never uses that kernel; a negative value uses it for everything it can run (tests).  Returns the
	 * previous value.  Process-wide. */
	AVHIP_API int avhip_set_small_problem_threshold(int workgroups);

	/* Tuning knob without a counterpart in the reference.  Products with a short k (at most 512 bytes per operand row: 1x1
	 * convolutions, the batched GEMM of non-fused Winograd) run on one of two engines: 0 (default) keeps the B operand (filters,
	 * transformed weights) in registers and streams only A through LDS; 1 passes both operands through LDS.  Returns the previous
	 * value.  Process-wide. */
	AVHIP_API int avhip_set_short_k_engine(int engine);

	/* Measurement aid without a counterpart in the reference: keeps every matrix core busy with register-resident
	 * 32x32 MFMAs of `dtype` (FLOAT16, BFLOAT16, INT8 or FLOAT32) and nothing else, so that a harness can time the rate the
	 * matrix cores sustain on this machine (clock under load included) next to the datasheet peak.  operands = 0: nearly
	 * all-zero operand bits (least switching activity, clock near boost); operands = 1: hashed bits shaped into finite
	 * numbers, several register sets in rotation (the switching activity, and so the clock, of real data).  Launches
	 * `workgroups` workgroups of 256 work-items, each wavefront issuing iterations * 8 MFMAs; sink receives one value per
	 * work-item (workgroups * 256 * 4 bytes).  Operations performed = workgroups * 4 * iterations * 8 * 2*32*32*k,
	 * k = 16 / 32 / 2 for 16-bit / int8 / fp32. */
	AVHIP_API int avhip_mfma_rate_probe(void *stream, int dtype, int workgroups, int iterations, int operands, void *sink);

	/* Measurement aid without a counterpart in the reference: a streaming kernel of known HBM traffic, so that a harness can
	 * put this machine's read, write and copy ceilings next to the datasheet bandwidth.  kind 0 reads `bytes` from src (dst
	 * must point to at least 4 writable bytes), kind 1 writes `bytes` to dst, kind 2 copies src to dst (2 * bytes of
	 * traffic).  16-byte aligned buffers; the last up to 16 KiB of a buffer may stay untouched. */
	AVHIP_API int avhip_stream_probe(void *stream, int kind, const void *src, void *dst, int64_t bytes);

#ifdef __cplusplus
}
#endif

#endif /* AVOCADO_HIP_KERNELS_H_ */
