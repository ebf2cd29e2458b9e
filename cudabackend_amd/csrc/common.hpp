/*
 * common.hpp -- device-side building blocks shared by every kernel file: storage types with
 * round-to-nearest-even conversion, bounds-aware vector access, activations.
 *
 * Behaviour carried over from the reference's Number<T> abstraction (the .cuh files under src/numbers): 16-bit tensors are
 * computed in fp32, loads and stores near the end of the channel dimension touch only the elements that exist.
 * Deliberate difference: bf16 stores round to nearest even (the reference truncates, src/numbers/bf16_number.cuh:40-43).
 */
#ifndef AVHIP_COMMON_HPP_
#define AVHIP_COMMON_HPP_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/avocado_hip_kernels.h"

namespace avhip
{
	enum DType
	{
		DT_UNKNOWN = 0, DT_UINT8, DT_INT8, DT_INT16, DT_INT32, DT_INT64, DT_FLOAT16, DT_BFLOAT16, DT_FLOAT32, DT_FLOAT64, DT_COMPLEX32, DT_COMPLEX64
	};
	enum Activation
	{
		ACT_LINEAR = 0, ACT_SIGMOID, ACT_TANH, ACT_RELU, ACT_SELU, ACT_ELU, ACT_EXPONENTIAL, ACT_SOFTPLUS, ACT_SOFTSIGN
	};

	struct bf16_t
	{
		uint16_t bits;
	};
	typedef _Float16 f16_t;

	__host__ __device__ inline float bf16_to_float(bf16_t v)
	{
		union
		{
			uint32_t u;
			float f;
		} c;
		c.u = static_cast<uint32_t>(v.bits) << 16;
		return c.f;
	}
	/* Round to nearest even.  On the device this is the single v_cvt_pk_bf16_f32 instruction of gfx950. */
	__host__ __device__ inline bf16_t float_to_bf16(float f)
	{
		bf16_t r;
#if defined(__HIP_DEVICE_COMPILE__)
		r.bits = __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));
#else
		union
		{
			uint32_t u;
			float f;
		} c;
		c.f = f;
		if ((c.u & 0x7FFFFFFFu) > 0x7F800000u) // NaN stays NaN
			r.bits = static_cast<uint16_t>((c.u >> 16) | 0x0040u);
		else
			r.bits = static_cast<uint16_t>((c.u + 0x7FFFu + ((c.u >> 16) & 1u)) >> 16);
#endif
		return r;
	}

	/* Storage type -> compute type and conversions. */
	template<typename T> struct Traits;
	template<> struct Traits<float>
	{
		typedef float compute;
		static constexpr int dtype = DT_FLOAT32;
		__host__ __device__ static float load(float v) { return v; }
		__host__ __device__ static float store(float v) { return v; }
	};
	template<> struct Traits<double>
	{
		typedef double compute;
		static constexpr int dtype = DT_FLOAT64;
		__host__ __device__ static double load(double v) { return v; }
		__host__ __device__ static double store(double v) { return v; }
	};
	template<> struct Traits<f16_t>
	{
		typedef float compute;
		static constexpr int dtype = DT_FLOAT16;
		__host__ __device__ static float load(f16_t v) { return static_cast<float>(v); }
		__host__ __device__ static f16_t store(float v) { return static_cast<f16_t>(v); }
	};
	template<> struct Traits<bf16_t>
	{
		typedef float compute;
		static constexpr int dtype = DT_BFLOAT16;
		__host__ __device__ static float load(bf16_t v) { return bf16_to_float(v); }
		__host__ __device__ static bf16_t store(float v) { return float_to_bf16(v); }
	};

	/* A naturally aligned pack of V elements of T moved with one memory instruction. */
	template<typename T, int V>
	struct alignas(sizeof(T) * V) Pack
	{
		T v[V];
	};

	/* Loads V consecutive elements starting at ptr into compute values; elements at or beyond `valid` are not touched
	 * and read as zero.  With allow_vector the pointer must be aligned to the pack whenever valid >= V. */
	template<typename T, int V, typename CT>
	__device__ inline void load_vec(const T *ptr, int valid, CT (&out)[V], bool allow_vector = true)
	{
		if (V > 1 && valid >= V && allow_vector)
		{
			const Pack<T, V> p = *reinterpret_cast<const Pack<T, V>*>(ptr);
#pragma unroll
			for (int i = 0; i < V; i++)
				out[i] = Traits<T>::load(p.v[i]);
		}
		else
		{
#pragma unroll
			for (int i = 0; i < V; i++)
				out[i] = (i < valid) ? static_cast<CT>(Traits<T>::load(ptr[i])) : static_cast<CT>(0);
		}
	}
	/* STREAM: the pack is written with a non-temporal store.  For tensors that the writing kernel never reads back this
	 * lets the caches drain them while the kernel still runs instead of at its end. */
	template<typename T, int V, typename CT, bool STREAM = false>
	__device__ inline void store_vec(T *ptr, int valid, const CT (&in)[V], bool allow_vector = true)
	{
		if (V > 1 && valid >= V && allow_vector)
		{
			typedef unsigned int words_t __attribute__((ext_vector_type((sizeof(T) * V + 3) / 4)));
			union
			{
				Pack<T, V> p;
				words_t words;
			} u;
#pragma unroll
			for (int i = 0; i < V; i++)
				u.p.v[i] = Traits<T>::store(in[i]);
			if (STREAM && sizeof(T) * V >= 4)
				__builtin_nontemporal_store(u.words, reinterpret_cast<words_t*>(ptr));
			else
				*reinterpret_cast<Pack<T, V>*>(ptr) = u.p;
		}
		else
		{
#pragma unroll
			for (int i = 0; i < V; i++)
				if (i < valid)
					ptr[i] = Traits<T>::store(in[i]);
		}
	}

	/* A whole 8- or 16-byte run stored "sc0 sc1 nt": streamed and written through to memory as the kernel runs.  Lines a kernel
	 * leaves dirty in L2 are written back when it ends, between it and the next dependent kernel; runs that cover only part
	 * of a cache line (8 int8 results per work-item) otherwise stay behind until then. */
	template<typename V>
	__device__ __forceinline__ void store_through(V *dst, const V &value)
	{
		static_assert(sizeof(V) == 8 || sizeof(V) == 16, "one dwordx2 or dwordx4 store");
		if constexpr (sizeof(V) == 8)
			asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" : : "v"(dst), "v"(value) : "memory");
		else
			asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" : : "v"(dst), "v"(value) : "memory");
	}
	/* The same written through without the streaming hint ("sc0 sc1") */
	template<typename V>
	__device__ __forceinline__ void store_through_plain(V *dst, const V &value)
	{
		static_assert(sizeof(V) == 8 || sizeof(V) == 16, "one dwordx2 or dwordx4 store");
		if constexpr (sizeof(V) == 8)
			asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" : : "v"(dst), "v"(value) : "memory");
		else
			asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(dst), "v"(value) : "memory");
	}

	/* Makes a wavefront-uniform 32-bit value live in a scalar register from here on.  Kernel arguments sit in memory and the
	 * compiler is free to re-load them wherever they are used; in fully unrolled epilogues that puts a scalar load and a
	 * wait in front of every store.  Passing the value through an empty asm statement makes it opaque, so it is loaded once.
	 * Not for pointers: a pointer that went through asm loses its address space and every access becomes a slow flat access. */
	template<typename T>
	__device__ __forceinline__ void keep_in_sgpr(T &v)
	{
		asm volatile("" : "+s"(v));
	}

	/* Issue priority of a wavefront inside the MFMA burst of one k-step, by how far the burst has come (slab = 32-byte part of
	 * the step).  Two wavefronts of different workgroups share a SIMD and its one matrix pipeline; at equal priority their
	 * bursts interleave, both finish late and both then wait for LDS together.  A wavefront that is further into its burst
	 * wins, so bursts run one after the other and each wavefront's loads and barrier fall under the other's MFMAs (measured
	 * on the 3x3 tile kernel: 3 % on the whole kernel against one fixed raised priority).  s_setprio takes an immediate. */
	__device__ __forceinline__ void burst_priority(int slab)
	{
		if (slab == 0)
			__builtin_amdgcn_s_setprio(1);
		else if (slab == 1)
			__builtin_amdgcn_s_setprio(2);
		else
			__builtin_amdgcn_s_setprio(3);
	}

	/* Workgroups of a grid are handed to the eight XCDs of the chip round-robin (workgroup b runs on XCD b % 8) and every
	 * XCD has its own L2.  Kernels whose neighbouring blocks of work share input (tiles with halos, pixel blocks whose filter
	 * windows overlap) renumber their workgroups so that each XCD owns a contiguous eighth of the blocks: workgroup b of nb
	 * takes block (b % 8) * (nb / 8) + b / 8; the last nb % 8 workgroups keep their own number. */
	__device__ inline unsigned int xcd_block(unsigned int b, unsigned int nb)
	{
		constexpr unsigned int XCDS = 8;
		const unsigned int per_xcd = nb / XCDS;
		return b < per_xcd * XCDS ? (b % XCDS) * per_xcd + b / XCDS : b;
	}

	/* Tile of a workgroup in a grid of (row blocks, column blocks): the column block (filters) runs fastest and each XCD owns a
	 * contiguous run, so the workgroups that read the same rows of the streamed operand run next to each other on one L2 and the
	 * operand comes from HBM once.  A grid walked in its own order (all row blocks of column block 0 first) reads it once per
	 * column block. */
	__device__ inline void xcd_tile(unsigned int &row_block, unsigned int &column_block)
	{
		const unsigned int t = xcd_block(blockIdx.y * gridDim.x + blockIdx.x, gridDim.x * gridDim.y);
		row_block = t / gridDim.y;
		column_block = t - row_block * gridDim.y;
	}

	/* Forward activations, src/activations.cuh:202-425 of the reference. */
	template<typename CT>
	__device__ inline CT activation_forward(int act, CT x)
	{
		switch (act)
		{
			default:
			case ACT_LINEAR:
				return x;
			case ACT_SIGMOID:
				return static_cast<CT>(1) / (static_cast<CT>(1) + exp(-x));
			case ACT_TANH:
				return tanh(x);
			case ACT_RELU:
				return x > static_cast<CT>(0) ? x : static_cast<CT>(0);
			case ACT_SELU:
				return static_cast<CT>(1.05070098) * (x >= static_cast<CT>(0) ? x : static_cast<CT>(1.67326324) * expm1(x));
			case ACT_ELU:
				return x >= static_cast<CT>(0) ? x : expm1(x);
			case ACT_EXPONENTIAL:
				return exp(x);
			case ACT_SOFTPLUS:
				return log1p(exp(x));
			case ACT_SOFTSIGN:
				return x / (fabs(x) + static_cast<CT>(1));
		}
	}

	__host__ inline int dtype_size(int dtype)
	{
		switch (dtype)
		{
			case DT_UINT8:
			case DT_INT8:
				return 1;
			case DT_INT16:
			case DT_FLOAT16:
			case DT_BFLOAT16:
				return 2;
			case DT_INT32:
			case DT_FLOAT32:
				return 4;
			case DT_INT64:
			case DT_FLOAT64:
			case DT_COMPLEX32:
				return 8;
			case DT_COMPLEX64:
				return 16;
			default:
				return 0;
		}
	}

	__host__ inline unsigned int ceil_div(int64_t a, int64_t b)
	{
		return static_cast<unsigned int>((a + b - 1) / b);
	}
	__host__ inline bool aligned_to(const void *p, size_t bytes)
	{
		return (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
	}
}

#endif /* AVHIP_COMMON_HPP_ */
