/*
 * avocado_hip_backend.h
 *
 * The drop-in boundary: the subset of Avocado's C backend API (include/Avocado/cuda_backend.h of the reference) that
 * the forward-convolution hot path needs, implemented for one AMD MI355X (gfx950).  Symbol names, argument order and
 * argument meaning are those of the reference so that a front-end written against the CUDA backend links against this
 * library unchanged; each declaration cites the reference line it replaces.  Functions of the reference header that
 * are not on the path are not exported.
 *
 * Conventions (include/Avocado/cuda_backend.h:22-52):
 *   - descriptors are passed by value; every pointer argument is HOST memory;
 *   - alpha-like scalars default to 1 and beta-like scalars to 0 when the pointer is null; their type is fp32 for
 *     integer / fp16 / bf16 / fp32 tensors and fp64 for fp64 tensors;
 *   - calls enqueue on the stream of the context and return; only copies issued on a default context block;
 *   - a memory descriptor that is not valid (0 or -1) where a bias or a residual is optional means "absent".
 * Tensors are NHWC, weights [K, R, S, C].  Padding is a signed input offset: "3x3, pad 1" is padding = {-1, -1}.
 */
#ifndef AVOCADO_HIP_BACKEND_H_
#define AVOCADO_HIP_BACKEND_H_

#include "avocado_backend_defs.h"

#ifdef __cplusplus
namespace avocado
{
	namespace backend
	{
		extern "C"
		{
#endif

			/* ---- device ------------------------------------------------------------------------------------------ */

			/* cuda_backend.h:58.  Number of visible GPUs, 0 on any error. */
			DLL_PUBLIC int cudaGetNumberOfDevices();
			/* cuda_backend.h:67.  result points to at least 256 bytes (name) or to an int32 / int64 / bool. */
			DLL_PUBLIC avStatus_t cudaGetDeviceProperty(avDeviceIndex_t index, avDeviceProperty_t propertyName, void *result);
			/* cuda_backend.h:76.  One GPU per process here: true only for from == to. */
			DLL_PUBLIC avStatus_t cudaIsCopyPossible(avDeviceIndex_t from, avDeviceIndex_t to, bool *result);

			/* ---- context ----------------------------------------------------------------------------------------- */

			/* cuda_backend.h:93.  A context owns one HIP stream of default priority on the device. */
			DLL_PUBLIC avStatus_t cudaCreateContextDescriptor(avContextDescriptor_t *result, avDeviceIndex_t deviceIndex);
			/* cuda_backend.h:104.  BAD_PARAM for an invalid or a default context. */
			DLL_PUBLIC avStatus_t cudaDestroyContextDescriptor(avContextDescriptor_t desc);
			/* cuda_backend.h:112.  The default context of a device uses the null stream; -1 for a bad device index. */
			DLL_PUBLIC avContextDescriptor_t cudaGetDefaultContext(avDeviceIndex_t deviceIndex);
			/* cuda_backend.h:122. */
			DLL_PUBLIC avStatus_t cudaSynchronizeWithContext(avContextDescriptor_t context);
			/* cuda_backend.h:133. */
			DLL_PUBLIC avStatus_t cudaIsContextReady(avContextDescriptor_t context, bool *result);

			/* ---- memory ------------------------------------------------------------------------------------------ */

			/* cuda_backend.h:151.  Allocates device memory (hipMalloc). */
			DLL_PUBLIC avStatus_t cudaCreateMemoryDescriptor(avMemoryDescriptor_t *result, avDeviceIndex_t deviceIndex, av_int64 sizeInBytes);
			/* cuda_backend.h:164.  Non-owning window into an owning block. */
			DLL_PUBLIC avStatus_t cudaCreateMemoryView(avMemoryDescriptor_t *result, const avMemoryDescriptor_t desc, av_int64 sizeInBytes,
					av_int64 offsetInBytes);
			/* cuda_backend.h:175. */
			DLL_PUBLIC avStatus_t cudaDestroyMemoryDescriptor(avMemoryDescriptor_t desc);
			/* cuda_backend.h:189.  pattern of 1, 2, 4, 8 or 16 bytes, or null for zeros. */
			DLL_PUBLIC avStatus_t cudaSetMemory(avContextDescriptor_t context, avMemoryDescriptor_t dst, av_int64 dstOffset, av_int64 dstSize,
					const void *pattern, av_int64 patternSize);
			/* cuda_backend.h:205. */
			DLL_PUBLIC avStatus_t cudaCopyMemory(avContextDescriptor_t context, avMemoryDescriptor_t dst, av_int64 dstOffset, const avMemoryDescriptor_t src,
					av_int64 srcOffset, av_int64 count);
			/* cuda_backend.h:211. */
			DLL_PUBLIC avStatus_t cudaCopyMemoryToHost(avContextDescriptor_t context, void *dst, const avMemoryDescriptor_t src, av_int64 srcOffset,
					av_int64 bytes);
			/* cuda_backend.h:217. */
			DLL_PUBLIC avStatus_t cudaCopyMemoryFromHost(avContextDescriptor_t context, avMemoryDescriptor_t dst, av_int64 dstOffset, const void *src,
					av_int64 bytes);
			/* cuda_backend.h:220,222.  Registering existing host memory is not available on this platform: NOT_SUPPORTED
			 * (BAD_PARAM for null), which callers treat as "stay pageable". */
			DLL_PUBLIC avStatus_t cudaPageLock(void *ptr, av_int64 count);
			DLL_PUBLIC avStatus_t cudaPageUnlock(void *ptr);

			/* ---- tensor descriptor ------------------------------------------------------------------------------- */

			/* cuda_backend.h:235,242,252,262. */
			DLL_PUBLIC avStatus_t cudaCreateTensorDescriptor(avTensorDescriptor_t *result);
			DLL_PUBLIC avStatus_t cudaDestroyTensorDescriptor(avTensorDescriptor_t desc);
			DLL_PUBLIC avStatus_t cudaSetTensorDescriptor(avTensorDescriptor_t desc, avDataType_t dtype, int nbDims, const int dimensions[]);
			DLL_PUBLIC avStatus_t cudaGetTensorDescriptor(avTensorDescriptor_t desc, avDataType_t *dtype, int *nbDims, int dimensions[]);

			/* ---- convolution descriptor -------------------------------------------------------------------------- */

			/* cuda_backend.h:743,750,764,779.  padding / strides / dilation may be null (0 / 1 / 1); paddingValue points to
			 * 16 bytes holding a scalar of the tensor dtype, or is null for zero. */
			DLL_PUBLIC avStatus_t cudaCreateConvolutionDescriptor(avConvolutionDescriptor_t *result);
			DLL_PUBLIC avStatus_t cudaDestroyConvolutionDescriptor(avConvolutionDescriptor_t desc);
			DLL_PUBLIC avStatus_t cudaSetConvolutionDescriptor(avConvolutionDescriptor_t desc, avConvolutionMode_t mode, int nbDims, const int padding[],
					const int strides[], const int dilation[], int groups, const void *paddingValue);
			DLL_PUBLIC avStatus_t cudaGetConvolutionDescriptor(avConvolutionDescriptor_t desc, avConvolutionMode_t *mode, int *nbDims, int padding[],
					int strides[], int dilation[], int *groups, void *paddingValue);

			/* ---- tensor operations on the path ------------------------------------------------------------------- */

			/* cuda_backend.h:281.  dst[i] = convert(src[i]); integers round to nearest even and saturate. */
			DLL_PUBLIC avStatus_t cudaChangeType(avContextDescriptor_t context, avMemoryDescriptor_t dst, avDataType_t dstType, const avMemoryDescriptor_t src,
					avDataType_t srcType, av_int64 elements);

			/* cuda_backend.h:380.  y = alpha1 * activation(alpha2 * x + b + beta1 * z) + beta2 * z + beta3 * y, b broadcast over
			 * the last dimension; fp16 / bf16 / fp32 (fp32 bias) and fp64 (fp64 bias). */
			DLL_PUBLIC avStatus_t cudaAddBias(avContextDescriptor_t context, const void *alpha1, const void *alpha2, const avTensorDescriptor_t xDesc,
					const avMemoryDescriptor_t xMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const avTensorDescriptor_t yDesc,
					avMemoryDescriptor_t yMem, const void *beta1, const void *beta2, const void *beta3, const avMemoryDescriptor_t zMem,
					avActivationType_t activation);

			/* cuda_backend.h:591.  y = alpha * activation(x * w + b) + beta * y with w, b broadcast over the trailing dimensions of
			 * x that they span (src/batchnorm.cu:28-48, 315-340).  fp16 / bf16 / fp32 tensors with fp32 parameters, fp64 with fp64. */
			DLL_PUBLIC avStatus_t cudaAffineForward(avContextDescriptor_t context, avActivationType_t activation, const avTensorDescriptor_t wDesc,
					const avMemoryDescriptor_t wMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha,
					const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const void *beta, const avTensorDescriptor_t yDesc,
					avMemoryDescriptor_t yMem);

			/* cuda_backend.h:612.  Batch normalisation with stored statistics: y = alpha * activation((x - mean) / sqrt(variance +
			 * epsilon) * scale + bias) + beta * y, evaluated as x * s + t with s = scale / sqrt(variance + epsilon), t = bias - mean * s
			 * (src/batchnorm.cu:51-69, 342-370).  Same data types as cudaAffineForward. */
			DLL_PUBLIC avStatus_t cudaBatchNormInference(avContextDescriptor_t context, avActivationType_t activation, const void *alpha,
					const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const void *beta, const avTensorDescriptor_t yDesc,
					avMemoryDescriptor_t yMem, const avTensorDescriptor_t scaleBiasMeanVarDesc, const avMemoryDescriptor_t scaleMem,
					const avMemoryDescriptor_t biasMem, const avMemoryDescriptor_t meanMem, const avMemoryDescriptor_t varianceMem, double epsilon);

			/* cuda_backend.h:442.  C = alpha * opA(A) opB(B) + beta * C, row-major.  fp16 / bf16 / fp32 / fp64, and
			 * int8 x int8 -> int32 with alpha, beta in {0, 1} and leading dimensions that are multiples of 4 (src/gemm.cpp:42-57). */
			DLL_PUBLIC avStatus_t cudaGemm(avContextDescriptor_t context, avGemmOperation_t aOp, avGemmOperation_t bOp, const void *alpha,
					const avTensorDescriptor_t aDesc, const avMemoryDescriptor_t aMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem,
					const void *beta, const avTensorDescriptor_t cDesc, avMemoryDescriptor_t cMem);
			/* cuda_backend.h:460.  Same per batch entry; the first dimension of every operand is the batch.  The (N, T) form is
			 * the matrix-core stage of non-fused Winograd.  The result of a 16-bit product may be fp32 (cDesc dtype). */
			DLL_PUBLIC avStatus_t cudaGemmBatched(avContextDescriptor_t context, avGemmOperation_t aOp, avGemmOperation_t bOp, const void *alpha,
					const avTensorDescriptor_t aDesc, const avMemoryDescriptor_t aMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem,
					const void *beta, const avTensorDescriptor_t cDesc, avMemoryDescriptor_t cMem);

			/* ---- convolution ------------------------------------------------------------------------------------- */

			/* cuda_backend.h:791.  rows[N*Ho*Wo, R*S*C] from x[N, H, W, C]; the descriptor's strides and dilations are honoured
			 * (Ho = (H - 2*padding - dilation*(R-1) - 1) / stride + 1; the reference's kernel assumes stride 1, dilation 1). */
			DLL_PUBLIC avStatus_t cudaIm2Row(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const avTensorDescriptor_t filterDesc,
					const avTensorDescriptor_t srcDesc, const avMemoryDescriptor_t srcMem, const avTensorDescriptor_t rowDesc, avMemoryDescriptor_t rowMem);

			/* cuda_backend.h:814 (defined in the reference under another name, src/conv2d_implicit_gemm.cu:303).
			 * y = activation(alpha1 * conv(x, w) + alpha2 * z + b) + beta * y by implicit GEMM on matrix cores.
			 *   fp16 / bf16 / fp32: y, z of the tensor dtype, b fp32.
			 *   int8 x, w: y int32 with an int32 (or absent) bias, alpha1 = 1, beta = 0, no z, LINEAR / RELU is exact integer
			 *   arithmetic; any other int8 combination casts the int32 sum to fp32, applies the formula in fp32 with an fp32
			 *   bias and stores y as int32 / int8 (round to nearest even, saturate) or fp32. */
			DLL_PUBLIC avStatus_t cudaConvolutionImplicitGemmForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config,
					const void *alpha1, const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc,
					const avMemoryDescriptor_t wMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2,
					const avTensorDescriptor_t zDesc, const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc,
					avMemoryDescriptor_t yMem, avActivationType_t activation);

			/* cuda_backend.h:840 (defined in the reference under another name, src/winograd_fused.cu:789).
			 * Same formula by one fused Winograd F(2x2, 3x3) kernel; 3x3, stride 1, dilation 1; fp16 / bf16 / fp32. */
			DLL_PUBLIC avStatus_t cudaConvolutionWinogradFusedForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config,
					const void *alpha1, const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc,
					const avMemoryDescriptor_t wMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2,
					const avTensorDescriptor_t zDesc, const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc,
					avMemoryDescriptor_t yMem, avActivationType_t activation);

			/* cuda_backend.h:856.  matrices[t*t, K, C] = G w G^T, transformSize m in {2, 4} for 3x3 and {2} for 5x5.  The dtype of
			 * the matrices is taken from matricesDesc: the tensor dtype, or FLOAT16 / FLOAT32 for 16-bit tensors. */
			DLL_PUBLIC avStatus_t cudaWinogradWeightTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
					const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem, const avTensorDescriptor_t matricesDesc,
					avMemoryDescriptor_t matricesMem);
			/* cuda_backend.h:871.  matrices[t*t, tiles, C] = B^T x-tile B with the descriptor's offsets and padding value. */
			DLL_PUBLIC avStatus_t cudaWinogradInputTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
					const avTensorDescriptor_t wDesc, const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem,
					const avTensorDescriptor_t matricesDesc, avMemoryDescriptor_t matricesMem);
			/* cuda_backend.h:895.  y = activation(alpha1 * A^T matrices A + alpha2 * z + b) + beta * y. */
			DLL_PUBLIC avStatus_t cudaWinogradOutputTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
					const avTensorDescriptor_t wDesc, const void *alpha1, const avTensorDescriptor_t matricesDesc, const avMemoryDescriptor_t matricesMem,
					const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem,
					const void *alpha2, const avTensorDescriptor_t zDesc, const avMemoryDescriptor_t zMem, const void *beta, avActivationType_t activation);

			/* cuda_backend.h:911.  Weight-gradient side: matrices[t*t, tiles, K] = G' dy-tile G'^T over non-overlapping
			 * transformSize x transformSize tiles of dy (src/winograd_nonfused.cu:963). */
			DLL_PUBLIC avStatus_t cudaWinogradGradientTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
					const avTensorDescriptor_t wDesc, const avTensorDescriptor_t dyDesc, const avMemoryDescriptor_t dyMem,
					const avTensorDescriptor_t matricesDesc, avMemoryDescriptor_t matricesMem);
			/* cuda_backend.h:927.  dw[K, r, r, C] = alpha * U' matrices[t*t, K, C] U'^T + beta * dw (src/winograd_nonfused.cu:983). */
			DLL_PUBLIC avStatus_t cudaWinogradUpdateTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
					const void *alpha, const avTensorDescriptor_t matricesDesc, const avMemoryDescriptor_t matricesMem, const void *beta,
					const avTensorDescriptor_t dwDesc, avMemoryDescriptor_t dwMem);

			/* Not in the reference header; NOT_SUPPORTED stubs at src/convolution.cu:30-99 of the reference.  Here they are the
			 * dispatcher a front-end calls per layer: it picks fused Winograd, non-fused Winograd (needs the workspace) or
			 * implicit GEMM from shape and dtype.  The workspace may be an invalid descriptor when the size query returned 0. */
			DLL_PUBLIC avStatus_t cudaGetConvolutionWorkspaceSize(avContextDescriptor_t context, const avConvolutionDescriptor_t config,
					const avTensorDescriptor_t xDesc, const avTensorDescriptor_t wDesc, const avTensorDescriptor_t bDesc, av_int64 *result);
			DLL_PUBLIC avStatus_t cudaConvolutionBiasActivationForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config,
					const void *alpha1, const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc,
					const avMemoryDescriptor_t wMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2,
					const avTensorDescriptor_t zDesc, const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc,
					avMemoryDescriptor_t yMem, const avActivationType_t activation, avMemoryDescriptor_t workspaceMem);
			DLL_PUBLIC avStatus_t cudaConvolutionForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const void *alpha,
					const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem,
					const void *beta, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem, avMemoryDescriptor_t workspaceMem);

			/* ---- additions without a counterpart in the reference ------------------------------------------------- */

			/* Quantised convolution with per-output-channel requantisation (the reference has no such step):
			 * y_int8 = saturate(round_nearest_even(float(conv_int32(x, w) + b_int32[k]) * scale_fp32[k])), after LINEAR or RELU
			 * applied to the int32 sum. */
			DLL_PUBLIC avStatus_t avhipConvolutionRequantForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config,
					const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem,
					const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const avTensorDescriptor_t scaleDesc,
					const avMemoryDescriptor_t scaleMem, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem, avActivationType_t activation);
			/* No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP graph capture,
			 * tight serving loops, harnesses that forbid hipMalloc): cudaConvolutionWinogradFusedForward with the transformed
			 * weights [16, K, C] (FLOAT16 for 16-bit tensors, FLOAT32 for fp32) kept in a fixed device array of
			 * AVHIP_NOALLOC_SCRATCH_BYTES inside the library instead of library-allocated memory; the weights are transformed on
			 * the context's stream in every call, nothing is cached, and no allocating routine is called.  Returns
			 * AVOCADO_STATUS_NOT_SUPPORTED when 16 * K * C matrix elements exceed the array.  Every call on a device shares that
			 * device's array: calls that overlap in time on one device (different contexts) race; calls on one context are ordered
			 * by its stream.  The first call on a device looks the array's address up (no allocation, but do it outside capture). */
#define AVHIP_NOALLOC_SCRATCH_BYTES (4u << 20)
			DLL_PUBLIC avStatus_t avhipConvolutionWinogradFusedForwardNoAlloc(avContextDescriptor_t context, const avConvolutionDescriptor_t config,
					const void *alpha1, const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc,
					const avMemoryDescriptor_t wMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2,
					const avTensorDescriptor_t zDesc, const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc,
					avMemoryDescriptor_t yMem, avActivationType_t activation);
			/* Interop for harnesses: the HIP stream (hipStream_t) of a context and the device address behind a memory
			 * descriptor. */
			DLL_PUBLIC avStatus_t avhipGetContextStream(avContextDescriptor_t context, void **stream);
			DLL_PUBLIC avStatus_t avhipGetMemoryPointer(avMemoryDescriptor_t mem, void **pointer);
			/* The Winograd plans (cudaConvolutionWinogradFusedForward, and the dispatcher where it picks one) keep transformed
			 * weights in library memory, one buffer per weight tensor, and transform again, into the same buffer and on the
			 * calling stream, when the weight bytes were written through this API since.  What callers must know:
			 *  - writes the library cannot see (through the raw address, or by a replayed graph): call avhipInvalidateCaches
			 *    afterwards.  It synchronises the device and frees every buffer, so no captured graph that contains a Winograd
			 *    call may be replayed after it; capture again.  The same holds after the weight block of such a call is destroyed.
			 *    Nothing else frees a buffer that a graph holds (see avhipSetWeightCacheBudget).
			 *  - under stream capture the library neither allocates nor transforms: a Winograd entry whose weights are not cached
			 *    and up to date returns AVOCADO_STATUS_BAD_ALLOC without launching anything (run the call once outside capture,
			 *    or use the NoAlloc entry); the dispatcher takes its implicit-GEMM plan instead.
			 *  - a call on another context than the one whose call transformed the weights waits for that transform by event.
			 * avhipGetWeightCacheState reports buffers held, their bytes and the number of weight transforms launched so far
			 * (any pointer may be null). */
			DLL_PUBLIC avStatus_t avhipInvalidateCaches(void);
			DLL_PUBLIC avStatus_t avhipGetWeightCacheState(av_int64 *entries, av_int64 *bytes, av_int64 *transforms);
			/* The cache keeps at most `bytes` of matrices (default 4 GiB): inserting a new tensor beyond that frees the least
			 * recently used buffers first, except those a captured graph holds (a buffer handed to a capturing stream stays until
			 * avhipInvalidateCaches or the destruction of its weight block: only those two invalidate graphs) and those a call on
			 * another thread has looked up and not yet launched its kernel for.  `previous`, when not null, receives the old limit.
			 * No counterpart in the reference, which has no such cache. */
			DLL_PUBLIC avStatus_t avhipSetWeightCacheBudget(av_int64 bytes, av_int64 *previous);
			/* The eviction rule of that cache applied to a made-up set of `count` buffers, without touching a device: buffer i has
			 * bytes[i] bytes, was last used at time last_use[i] and carries flags[i] (1: held by a graph, 2: looked up by a call
			 * that has not launched yet).  evicted[i] is set to 1 for every buffer the rule frees to make room for `incoming` more
			 * bytes under `budget`, 0 otherwise.  For host-side tests of the policy. */
			DLL_PUBLIC avStatus_t avhipWeightCachePolicyProbe(int count, const av_int64 *bytes, const av_int64 *last_use, const int *flags, av_int64 budget,
					av_int64 incoming, int *evicted);

#ifdef __cplusplus
		} /* extern "C" */
	} /* namespace backend */
} /* namespace avocado */
#endif

#endif /* AVOCADO_HIP_BACKEND_H_ */
