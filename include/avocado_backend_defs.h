/*
 * avocado_backend_defs.h
 *
 * Types, enumerations and status codes of Avocado's C backend API, restated from how the reference
 * backend uses them.  The original header (Avocado/backend_defs.h, included at
 * include/Avocado/cuda_backend.h:11 of the reference) belongs to a sibling project that is not part of
 * the reference checkout, so only the NAMES are pinned; the integer value of every enumerator and the
 * bit layout of the descriptor handles below are this build's own choice.  A maintainer who links this
 * library into Avocado replaces this one file by the original and rebuilds: nothing else in the
 * library depends on the numeric values.
 */
#ifndef AVOCADO_BACKEND_DEFS_H_
#define AVOCADO_BACKEND_DEFS_H_

#include <stdint.h>
#ifndef __cplusplus
#  include <stdbool.h>
#endif

#ifndef DLL_PUBLIC
#  define DLL_PUBLIC __attribute__((visibility("default")))
#endif

#define AVOCADO_MAX_TENSOR_DIMENSIONS 8 /* Array8D, src/tensor_op.cu:67-71 of the reference */

#ifdef __cplusplus
namespace avocado
{
	namespace backend
	{
#endif

		typedef int64_t av_int64;
		typedef int avDeviceIndex_t;

		/* Opaque handles, passed by value; -1 is the invalid handle (src/descriptors.cu:212). */
		typedef av_int64 avContextDescriptor_t;
		typedef av_int64 avMemoryDescriptor_t;
		typedef av_int64 avTensorDescriptor_t;
		typedef av_int64 avConvolutionDescriptor_t;

		/* Status codes used by the reference: src/utilities.hpp:28-51, src/descriptors.cu:64,68,105. */
		typedef enum
		{
			AVOCADO_STATUS_SUCCESS = 0,
			AVOCADO_STATUS_ALLOC_FAILED,
			AVOCADO_STATUS_FREE_FAILED,
			AVOCADO_STATUS_BAD_ALLOC,
			AVOCADO_STATUS_BAD_PARAM,
			AVOCADO_STATUS_ARCH_MISMATCH,
			AVOCADO_STATUS_INTERNAL_ERROR,
			AVOCADO_STATUS_NOT_SUPPORTED,
			AVOCADO_STATUS_UNSUPPORTED_DATATYPE,
			AVOCADO_STATUS_EXECUTION_FAILED,
			AVOCADO_STATUS_INSUFFICIENT_DRIVER,
			AVOCADO_STATUS_DEVICE_TYPE_MISMATCH
		} avStatus_t;

		/* Data types: src/conversions.cu:270-301. */
		typedef enum
		{
			AVOCADO_DTYPE_UNKNOWN = 0,
			AVOCADO_DTYPE_UINT8,
			AVOCADO_DTYPE_INT8,
			AVOCADO_DTYPE_INT16,
			AVOCADO_DTYPE_INT32,
			AVOCADO_DTYPE_INT64,
			AVOCADO_DTYPE_FLOAT16,
			AVOCADO_DTYPE_BFLOAT16,
			AVOCADO_DTYPE_FLOAT32,
			AVOCADO_DTYPE_FLOAT64,
			AVOCADO_DTYPE_COMPLEX32,
			AVOCADO_DTYPE_COMPLEX64
		} avDataType_t;

		/* Activations: src/activations.cuh:436-454. */
		typedef enum
		{
			AVOCADO_ACTIVATION_LINEAR = 0,
			AVOCADO_ACTIVATION_SIGMOID,
			AVOCADO_ACTIVATION_TANH,
			AVOCADO_ACTIVATION_RELU,
			AVOCADO_ACTIVATION_SELU,
			AVOCADO_ACTIVATION_ELU,
			AVOCADO_ACTIVATION_EXPONENTIAL,
			AVOCADO_ACTIVATION_SOFTPLUS,
			AVOCADO_ACTIVATION_SOFTSIGN
		} avActivationType_t;

		/* CONVOLUTION: kernel applied as stored; CROSS_CORRELATION: kernel rotated by 180 degrees
		 * (src/winograd_nonfused.cu:616,279-282, app/CudaBackend.cu:170-179). */
		typedef enum
		{
			AVOCADO_CONVOLUTION_MODE = 0,
			AVOCADO_CROSS_CORRELATION_MODE
		} avConvolutionMode_t;

		typedef enum
		{
			AVOCADO_GEMM_OPERATION_N = 0,
			AVOCADO_GEMM_OPERATION_T
		} avGemmOperation_t;

		/* Device properties: src/cuda_properties.cpp:52-96. */
		typedef enum
		{
			AVOCADO_DEVICE_NAME = 0,
			AVOCADO_DEVICE_PROCESSOR_COUNT,
			AVOCADO_DEVICE_MEMORY,
			AVOCADO_DEVICE_SUPPORTS_HALF_PRECISION,
			AVOCADO_DEVICE_SUPPORTS_BFLOAT16,
			AVOCADO_DEVICE_SUPPORTS_SINGLE_PRECISION,
			AVOCADO_DEVICE_SUPPORTS_DOUBLE_PRECISION,
			AVOCADO_DEVICE_SUPPORTS_SSE,
			AVOCADO_DEVICE_SUPPORTS_SSE2,
			AVOCADO_DEVICE_SUPPORTS_SSE3,
			AVOCADO_DEVICE_SUPPORTS_SSSE3,
			AVOCADO_DEVICE_SUPPORTS_SSE41,
			AVOCADO_DEVICE_SUPPORTS_SSE42,
			AVOCADO_DEVICE_SUPPORTS_AVX,
			AVOCADO_DEVICE_SUPPORTS_AVX2,
			AVOCADO_DEVICE_SUPPORTS_AVX512_F,
			AVOCADO_DEVICE_SUPPORTS_AVX512_VL_BW_DQ,
			AVOCADO_DEVICE_SUPPORTS_DP4A,
			AVOCADO_DEVICE_ARCH_MAJOR,
			AVOCADO_DEVICE_ARCH_MINOR,
			AVOCADO_DEVICE_SUPPORTS_TENSOR_CORES
		} avDeviceProperty_t;

#ifdef __cplusplus
	} /* namespace backend */
} /* namespace avocado */
#endif

#endif /* AVOCADO_BACKEND_DEFS_H_ */
