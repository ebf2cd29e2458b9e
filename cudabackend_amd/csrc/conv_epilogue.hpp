/*
 * conv_epilogue.hpp -- what happens to a convolution accumulator on its way to y, shared by the implicit-GEMM kernels.
 *
 *   y = activation(alpha1 * conv + bias[k] + alpha2 * z) + beta * y
 * in the operation order of the reference's epilogue (src/winograd_nonfused.cu:407-417 of the reference): scale, add bias,
 * add the scaled residual, activate, add the scaled old output, store.  The MFMA engine hands every work-item four
 * consecutive output filters of one output pixel at a time; the per-filter constants of those four columns (bias, requant
 * scale) never change for a work-item, so they are loaded once, before the k loop, and not in the store loop.
 */
#ifndef AVHIP_CONV_EPILOGUE_HPP_
#define AVHIP_CONV_EPILOGUE_HPP_

#include "common.hpp"

namespace avhip
{
	/* How a kernel instance treats the activation.  ACT_SIMPLE instances are launched only for LINEAR and RELU and pay one
	 * v_max_f32 per element behind a wavefront-uniform branch; ACT_ANY instances switch over all nine functions.  The split is
	 * made on the host, per launch: a per-element switch in one kernel would make the compiler evaluate every transcendental
	 * and select. */
	constexpr int ACT_SIMPLE = -2;
	constexpr int ACT_ANY = -1;
	__host__ inline bool is_simple_activation(int activation)
	{
		return activation == ACT_LINEAR || activation == ACT_RELU;
	}
	template<int ACT, typename CT>
	__device__ __forceinline__ CT activate(int activation, CT x)
	{
		if (ACT == ACT_SIMPLE)
			return (activation == ACT_RELU && x < static_cast<CT>(0)) ? static_cast<CT>(0) : x;
		return activation_forward<CT>(activation, x);
	}
	__device__ inline int round_saturate(float v, float lo, float hi)
	{
		if (!(v == v))
			return 0;
		float r = rintf(v);
		r = r < lo ? lo : r;
		if (r >= 2147483648.0f) /* hi = 2^31 stands for INT32_MAX, which fp32 cannot hold */
			return 2147483647;
		r = r > hi ? hi : r;
		return static_cast<int>(r);
	}

	/* Floating tensors: TE in, TE out, fp32 bias, fp32 arithmetic, one round-to-nearest-even on store. */
	template<typename TE>
	struct FloatEpilogue
	{
		typedef float scalar_t;
		/* widest run of filters one work-item can store with a single 16-byte instruction */
		static constexpr int wide = sizeof(TE) >= 4 ? 4 : 8;
		template<int W> struct ColumnsT
		{
			float bias[W];
		};
		typedef ColumnsT<4> Columns;
		const float *bias;
		const TE *z;
		TE *y;
		float alpha1, alpha2, beta;
		int activation, K;
		bool vec; /* y / z rows may be accessed as 4-element vectors */

		/* call once on the kernel's copy before the k loop: the members are then read from scalar registers */
		__device__ __forceinline__ void pin()
		{
			keep_in_sgpr(alpha1);
			keep_in_sgpr(alpha2);
			keep_in_sgpr(beta);
			keep_in_sgpr(activation);
			keep_in_sgpr(K);
		}
		template<int W>
		__device__ __forceinline__ void load_columns(int k, ColumnsT<W> &c) const
		{
#pragma unroll
			for (int q = 0; q < W; q++)
				c.bias[q] = (bias != nullptr && k + q < K) ? bias[k + q] : 0.0f;
		}
		/* The same constants requested with 16-byte buffer loads and nothing else: filters past the last one and an absent bias
		 * read zeros through the buffer's bounds, so no instruction between here and the epilogue depends on the loaded values
		 * and a kernel does not wait for them before its k loop (a select on a loaded value would sit in the prologue and wait
		 * there).  k a multiple of 4, bias 16-byte aligned; finish_columns() before the first use. */
		template<int W>
		__device__ __forceinline__ void request_columns(int k, ColumnsT<W> &c) const
		{
			static_assert(W % 4 == 0, "whole 16-byte runs");
			const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(bias), 0, bias != nullptr ? K * 4 : 0, 0x00020000);
#pragma unroll
			for (int part = 0; part < W / 4; part++)
			{
				typedef float f32x4 __attribute__((ext_vector_type(4)));
				const f32x4 v = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rb, (k + 4 * part) * 4, 0, 0));
#pragma unroll
				for (int q = 0; q < 4; q++)
					c.bias[4 * part + q] = v[q];
			}
		}
		template<int W>
		__device__ __forceinline__ void finish_columns(ColumnsT<W>&) const
		{
		}
		/* the same constants out of a table of one-filter records (a kernel that walks several filter blocks stages
		 * load_columns(k, table[k]) for every k in LDS once) */
		template<int W>
		__device__ static __forceinline__ void pick_columns(const ColumnsT<1> *table, int k, ColumnsT<W> &c)
		{
#pragma unroll
			for (int q = 0; q < W; q++)
				c.bias[q] = table[k + q].bias[0];
		}
		/* p: index of the output pixel (row of y), k: first of the W filters.  VEC instances require whole, aligned vectors. */
		template<int ACT, bool VEC = false>
		__device__ __forceinline__ void store(int64_t p, int k, const float (&v)[4], const Columns &c) const
		{
			store_at<ACT, VEC, 4>(p * K + k, k, v, c);
		}
		/* W values of the residual z, fetched ahead of the epilogue by callers that know their rows early: a load issued
		 * inside the store loop cannot pass the stores before it (y and z may alias) and its latency adds up row by row. */
		template<int W> struct Residual
		{
			Pack<TE, W> raw;
		};
		template<int W>
		__device__ __forceinline__ void load_residual(int64_t idx, Residual<W> &r) const
		{
			if (z != nullptr)
				r.raw = *reinterpret_cast<const Pack<TE, W>*>(z + idx); /* whole, aligned runs only (VEC callers) */
		}
		/* t = [max(0, .)] (alpha1 * v + bias [+ alpha2 * zv]); max(0, x) as the reference writes ReLU (src/activations.cuh:274-293) */
		template<bool RELU, bool HAS_Z, int W>
		__device__ __forceinline__ void combine(float (&t)[W], const float (&v)[W], const ColumnsT<W> &c, const float (&zv)[W]) const
		{
#pragma unroll
			for (int q = 0; q < W; q++)
			{
				float r = alpha1 * v[q] + c.bias[q];
				if (HAS_Z)
					r += alpha2 * zv[q];
				t[q] = RELU ? __builtin_fmaxf(r, 0.0f) : r;
			}
		}
		/* The arithmetic of store_at without its store.  `readable`: the run exists in y and z (callers that store
		 * unconditionally compute rows past the end of the tensor on zeros). */
		template<int ACT, bool VEC, int W>
		__device__ __forceinline__ void values(float (&t)[W], bool readable, int64_t idx, int k, const float (&v)[W], const ColumnsT<W> &c,
				const Residual<W> *fetched) const
		{
			const bool vec = VEC || this->vec;
			const int valid = VEC ? W : K - k;
			/* ReLU sits in the same straight-line block as the multiply-add that feeds it: the compiler then knows the
			 * operand is an arithmetic result (never a signalling NaN) and emits one bare v_max_f32 per element */
			const bool relu = ACT == ACT_SIMPLE && activation == ACT_RELU;
			if (z != nullptr)
			{
				float zv[W];
				if (fetched != nullptr)
				{
#pragma unroll
					for (int q = 0; q < W; q++)
						zv[q] = Traits<TE>::load(fetched->raw.v[q]);
				}
				else if (readable)
					load_vec<TE, W, float>(z + idx, valid, zv, vec);
				else
				{
#pragma unroll
					for (int q = 0; q < W; q++)
						zv[q] = 0.0f;
				}
				if (relu)
					combine<true, true, W>(t, v, c, zv);
				else
					combine<false, true, W>(t, v, c, zv);
			}
			else
			{
				if (relu)
					combine<true, false, W>(t, v, c, v);
				else
					combine<false, false, W>(t, v, c, v);
			}
			if (ACT != ACT_SIMPLE)
			{
#pragma unroll
				for (int q = 0; q < W; q++)
					t[q] = activation_forward<float>(activation, t[q]);
			}
			if (beta != 0.0f && readable)
			{
				float yv[W];
				load_vec<TE, W, float>(y + idx, valid, yv, vec);
#pragma unroll
				for (int q = 0; q < W; q++)
					t[q] += beta * yv[q];
			}
		}
		/* idx: element index of (pixel, filter k) in y and z, for callers that keep it cheaper than p * K + k */
		template<int ACT, bool VEC = false, int W = 4>
		__device__ __forceinline__ void store_at(int64_t idx, int k, const float (&v)[W], const ColumnsT<W> &c, const Residual<W> *fetched = nullptr) const
		{
			static_assert(VEC || W == 4, "`vec` vouches for 4-element vectors only; wider runs are for callers that checked");
			float t[W];
			values<ACT, VEC, W>(t, true, idx, k, v, c, fetched);
			store_vec<TE, W, float, VEC>(y + idx, VEC ? W : K - k, t, VEC || this->vec);
		}
		/* For kernels that walk many tiles and must not have a store behind a condition (vector-memory operations complete in
		 * order and are counted statically: after a conditional store every later wait for an older load also waits for the
		 * store): the W results as 16 bytes handed to `sink` exactly once, whether or not the run exists; the caller's sink
		 * drops runs that do not (a buffer store at an out-of-range offset).  LINEAR / RELU, whole aligned runs. */
		static constexpr bool masked_stores = true;
		static constexpr int out_bytes = sizeof(TE);
		__device__ __forceinline__ char *out() const { return reinterpret_cast<char*>(y); }
		/* The same hand-over with everything about the call decided at compile time (ReLU or not, residual or not, beta = 0,
		 * the residual already fetched): no branch at all, for epilogues that run eight of these per work-item back to back
		 * and are otherwise paced by the branches between them. */
		template<bool RELU, bool HAS_Z, int W, typename Sink>
		__device__ __forceinline__ void store_fast(const float (&v)[W], const ColumnsT<W> &c, const Residual<W> &fetched, const Sink &sink) const
		{
			static_assert(W * sizeof(TE) == 16, "one 16-byte run");
			float t[W], zv[W];
#pragma unroll
			for (int q = 0; q < W; q++)
				zv[q] = HAS_Z ? Traits<TE>::load(fetched.raw.v[q]) : 0.0f;
			combine<RELU, HAS_Z, W>(t, v, c, zv);
			typedef unsigned int words_t __attribute__((ext_vector_type(4)));
			union
			{
				Pack<TE, W> p;
				words_t words;
			} u;
#pragma unroll
			for (int q = 0; q < W; q++)
				u.p.v[q] = Traits<TE>::store(t[q]);
			sink(u.words);
		}
		/* 16-bit tensors: a caller that walks tiles may fetch the residual of a pass of rows ahead (Residual, one 16-byte run
		 * each) and hand it in; the fp32 kernels have no registers left for that */
		static constexpr bool residual_ahead = sizeof(TE) == 2;
		__device__ __forceinline__ const char *residual() const { return reinterpret_cast<const char*>(z); }
		template<int W, typename Sink>
		__device__ __forceinline__ void store_masked(bool exists, int64_t idx, int k, const float (&v)[W], const ColumnsT<W> &c, const Sink &sink,
				const Residual<W> *fetched = nullptr) const
		{
			static_assert(W * sizeof(TE) == 16, "one 16-byte run");
			float t[W];
			values<ACT_SIMPLE, true, W>(t, exists, idx, k, v, c, fetched);
			typedef unsigned int words_t __attribute__((ext_vector_type(4)));
			union
			{
				Pack<TE, W> p;
				words_t words;
			} u;
#pragma unroll
			for (int q = 0; q < W; q++)
				u.p.v[q] = Traits<TE>::store(t[q]);
			sink(u.words);
		}
	};

	template<int N> struct Words
	{
		typedef int type __attribute__((ext_vector_type(N)));
	};
	template<> struct Words<1>
	{
		typedef int type;
	};

	enum Int8Mode
	{
		I8_EXACT = 0, /* y int32 = act(sum + bias_i32)                                   */
		I8_REQUANT, /* y int8  = sat(rne(float(act(sum + bias_i32)) * scale[k]))        */
		I8_FLOAT_I32, /* float epilogue, y int32                                         */
		I8_FLOAT_I8, /* float epilogue, y int8                                           */
		I8_FLOAT_F32 /* float epilogue, y fp32                                           */
	};

	/* int8 x int8 -> int32 sums.  EXACT and REQUANT add an int32 bias in integer arithmetic; the FLOAT modes follow the
	 * header's convention for integer tensors: cast to fp32, scale and add in fp32 (every step rounded once, no fused
	 * multiply-add), cast back with round-to-nearest-even and saturation. */
	template<int MODE>
	struct Int8Epilogue
	{
		typedef int scalar_t;
		static constexpr int wide = MODE == I8_REQUANT ? 8 : 4;
		template<int W> struct ColumnsT
		{
			int ibias[W];
			float fbias[W];
			float scale[W];
		};
		typedef ColumnsT<4> Columns;
		const void *bias, *z;
		void *y;
		const float *scale;
		float alpha1, alpha2, beta;
		int activation, K;
		bool vec;
		bool through; /* int8 results are written through (store_at); set by kernels whose workgroups store parts of cache lines */

		__device__ __forceinline__ void pin()
		{
			keep_in_sgpr(alpha1);
			keep_in_sgpr(alpha2);
			keep_in_sgpr(beta);
			keep_in_sgpr(activation);
			keep_in_sgpr(K);
		}
		template<int W>
		__device__ __forceinline__ void load_columns(int k, ColumnsT<W> &c) const
		{
#pragma unroll
			for (int q = 0; q < W; q++)
			{
				const bool in = k + q < K;
				c.ibias[q] = (MODE <= I8_REQUANT && bias != nullptr && in) ? static_cast<const int*>(bias)[k + q] : 0;
				c.fbias[q] = (MODE > I8_REQUANT && bias != nullptr && in) ? static_cast<const float*>(bias)[k + q] : 0.0f;
				/* Requantisation multiplies a finite fp32 value by the scale and clamps.  A NaN scale gives NaN -> 0 for every
				 * sum, exactly what a zero scale gives; an infinite scale saturates every non-zero sum and gives NaN -> 0 for
				 * a zero sum, exactly what the largest finite scale gives.  Replacing them here, once per filter, leaves the
				 * per-element path free of NaN handling. */
				float sc = (MODE == I8_REQUANT && in) ? scale[k + q] : 0.0f;
				sc = (sc == sc) ? sc : 0.0f;
				sc = sc > 3.0e38f ? 3.0e38f : (sc < -3.0e38f ? -3.0e38f : sc);
				c.scale[q] = sc;
			}
		}
		/* Requested with 16-byte buffer loads and left untouched until finish_columns() (see FloatEpilogue::request_columns):
		 * k a multiple of 4, bias and scale 16-byte aligned. */
		template<int W>
		__device__ __forceinline__ void request_columns(int k, ColumnsT<W> &c) const
		{
			static_assert(W % 4 == 0, "whole 16-byte runs");
			const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(bias), 0, bias != nullptr ? K * 4 : 0, 0x00020000);
			const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(scale), 0, (MODE == I8_REQUANT && scale != nullptr) ? K * 4 : 0,
					0x00020000);
#pragma unroll
			for (int part = 0; part < W / 4; part++)
			{
				typedef float f32x4 __attribute__((ext_vector_type(4)));
				typedef int i32x4 __attribute__((ext_vector_type(4)));
				const auto raw = __builtin_amdgcn_raw_buffer_load_b128(rb, (k + 4 * part) * 4, 0, 0);
#pragma unroll
				for (int q = 0; q < 4; q++)
				{
					c.ibias[4 * part + q] = MODE <= I8_REQUANT ? __builtin_bit_cast(i32x4, raw)[q] : 0;
					c.fbias[4 * part + q] = MODE > I8_REQUANT ? __builtin_bit_cast(f32x4, raw)[q] : 0.0f;
				}
				if (MODE == I8_REQUANT)
				{
					const f32x4 sv = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, (k + 4 * part) * 4, 0, 0));
#pragma unroll
					for (int q = 0; q < 4; q++)
						c.scale[4 * part + q] = sv[q];
				}
				else
				{
#pragma unroll
					for (int q = 0; q < 4; q++)
						c.scale[4 * part + q] = 0.0f;
				}
			}
		}
		/* the clean-up of the scales that load_columns does at once (NaN -> 0, infinities -> the largest finite value) */
		template<int W>
		__device__ __forceinline__ void finish_columns(ColumnsT<W> &c) const
		{
			if (MODE == I8_REQUANT)
			{
#pragma unroll
				for (int q = 0; q < W; q++)
				{
					float sc = c.scale[q];
					sc = (sc == sc) ? sc : 0.0f;
					c.scale[q] = sc > 3.0e38f ? 3.0e38f : (sc < -3.0e38f ? -3.0e38f : sc);
				}
			}
		}
		template<int W>
		__device__ static __forceinline__ void pick_columns(const ColumnsT<1> *table, int k, ColumnsT<W> &c)
		{
#pragma unroll
			for (int q = 0; q < W; q++)
			{
				c.ibias[q] = table[k + q].ibias[0];
				c.fbias[q] = table[k + q].fbias[0];
				c.scale[q] = table[k + q].scale[0];
			}
		}
		template<int ACT, bool VEC = false>
		__device__ __forceinline__ void store(int64_t p, int k, const int (&v)[4], const Columns &c) const
		{
			store_at<ACT, VEC, 4>(p * K + k, k, v, c);
		}
		template<int W> struct Residual /* nothing is fetched ahead on the integer paths */
		{
		};
		template<int W>
		__device__ __forceinline__ void load_residual(int64_t, Residual<W>&) const
		{
		}
		/* EXACT / REQUANT: act(sum + bias) in integer arithmetic */
		template<int W>
		__device__ __forceinline__ void integer_values(int (&t)[W], const int (&v)[W], const ColumnsT<W> &c) const
		{
			/* one v_max_i32 against a scalar either way (hidden from the optimiser, which would otherwise turn it back
			 * into a maximum and a select per element) */
			int floor = activation == ACT_RELU ? 0 : -2147483647 - 1;
			keep_in_sgpr(floor);
#pragma unroll
			for (int q = 0; q < W; q++)
			{
				t[q] = v[q] + c.ibias[q];
				t[q] = t[q] < floor ? floor : t[q];
			}
		}
		/* REQUANT: sat_i8(rne(float(t) * scale)), four results per 32-bit word.
		 * Clamping to the integers -128 and 127 commutes with rounding to an integer, so the product is clamped
		 * first; adding 1.5 * 2^23 then rounds it to nearest even in the adder (the sum's unit in the last place is 1)
		 * and leaves the two's-complement byte in the low 8 bits of the sum: no rint, no conversion.  Three byte
		 * permutes gather four such bytes into a word. */
		template<int W>
		__device__ __forceinline__ void requantise(unsigned int (&words)[W / 4], const int (&t)[W], const ColumnsT<W> &c) const
		{
#pragma clang fp contract(off)
#pragma unroll
			for (int part = 0; part < W / 4; part++)
			{
				unsigned int bits[4];
#pragma unroll
				for (int q = 0; q < 4; q++)
				{
					const float product = static_cast<float>(t[4 * part + q]) * c.scale[4 * part + q];
					const float rounded = __builtin_amdgcn_fmed3f(product, -128.0f, 127.0f) + 12582912.0f;
					bits[q] = __builtin_bit_cast(unsigned int, rounded);
				}
				const unsigned int lo = __builtin_amdgcn_perm(bits[1], bits[0], 0x0c0c0400u);
				const unsigned int hi = __builtin_amdgcn_perm(bits[3], bits[2], 0x0c0c0400u);
				words[part] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
			}
		}
		/* no unconditional hand-over of runs (FloatEpilogue::store_masked) here: measured on the 1x1 layer of config 4 it
		 * made the int32-output kernel 5 % slower and left the requantising one unchanged */
		static constexpr bool masked_stores = false;
		template<int ACT, bool VEC = false, int W = 4>
		__device__ __forceinline__ void store_at(int64_t idx, int k, const int (&v)[W], const ColumnsT<W> &c, const Residual<W>* = nullptr) const
		{
			/* every fp32 operation below rounds exactly once: a * b + c must not become a fused multiply-add.  The pragma
			 * governs the expressions written in this block, which is why they use plain operators and no intrinsics. */
#pragma clang fp contract(off)
			static_assert(VEC || W == 4, "`vec` vouches for 4-element vectors only; wider runs are for callers that checked");
			const bool vec = VEC || this->vec;
			const int valid = VEC ? W : K - k;
			if (MODE == I8_EXACT || MODE == I8_REQUANT)
			{
				int t[W];
				integer_values<W>(t, v, c);
				/* int32 results (16 bytes per work-item, whole cache lines per row) leave as non-temporal vector stores: the
				 * kernel never reads y back, so the caches may drain it while the kernel runs.  int8 results of a workgroup that
				 * writes whole lines (the 1x1 kernels) leave as ordinary stores, 8 bytes per work-item, which L2 puts together:
				 * 7.7 us on config 4 (9.8 us written through, 7.6 us with the non-temporal hint), but a layer that writes 206 MB
				 * takes 95 us this way against 221 us with the hint.  Where a workgroup's row of int8 results is part of a cache
				 * line (64 filters of the tile kernel) they are written through, or the partial lines wait in L2 for the
				 * write-back at the end of the kernel (config 4, requantised 3x3 layer: 17.0 -> 14.8 us; int32 results there:
				 * 14.6 -> 16.6 us) */
				typedef typename Words<W / 4>::type words_t; /* W int8 values as 32-bit words */
				if (MODE == I8_EXACT)
				{
					int *dst = static_cast<int*>(y) + idx;
					if (vec && valid >= W)
					{
#pragma unroll
						for (int part = 0; part < W / 4; part++)
						{
							typedef int i32x4 __attribute__((ext_vector_type(4)));
							const i32x4 pack = { t[4 * part], t[4 * part + 1], t[4 * part + 2], t[4 * part + 3] };
							__builtin_nontemporal_store(pack, reinterpret_cast<i32x4*>(dst) + part);
						}
					}
					else
					{
#pragma unroll
						for (int q = 0; q < W; q++)
							if (q < valid)
								dst[q] = t[q];
					}
				}
				else
				{
					union
					{
						int8_t b[W];
						unsigned int u[W / 4];
						words_t w;
					} o;
					requantise<W>(o.u, t, c);
					int8_t *dst = static_cast<int8_t*>(y) + idx;
					if (vec && valid >= W)
					{
						if constexpr (sizeof(words_t) >= 8)
						{
							if (through)
								store_through_plain(reinterpret_cast<words_t*>(dst), o.w); /* (13.4-13.6 us on config 4 against 13.8 with the streaming hint as well) */
							else
								*reinterpret_cast<words_t*>(dst) = o.w;
						}
						else
							__builtin_nontemporal_store(o.w, reinterpret_cast<words_t*>(dst));
					}
					else
					{
#pragma unroll
						for (int q = 0; q < W; q++)
							if (q < valid)
								dst[q] = o.b[q];
					}
				}
			}
			else
			{
#pragma unroll
				for (int q = 0; q < W; q++)
				{
					if (q >= valid)
						continue;
					float t = alpha1 * static_cast<float>(v[q]);
					if (bias != nullptr)
						t = t + c.fbias[q];
					if (z != nullptr)
					{
						const float zv = MODE == I8_FLOAT_I32 ? static_cast<float>(static_cast<const int*>(z)[idx + q]) :
											MODE == I8_FLOAT_I8 ? static_cast<float>(static_cast<const int8_t*>(z)[idx + q]) : static_cast<const float*>(z)[idx + q];
						t = t + alpha2 * zv;
					}
					t = activate<ACT, float>(activation, t);
					if (beta != 0.0f)
					{
						const float yv = MODE == I8_FLOAT_I32 ? static_cast<float>(static_cast<int*>(y)[idx + q]) :
											MODE == I8_FLOAT_I8 ? static_cast<float>(static_cast<int8_t*>(y)[idx + q]) : static_cast<float*>(y)[idx + q];
						t = t + beta * yv;
					}
					if (MODE == I8_FLOAT_I32)
						static_cast<int*>(y)[idx + q] = round_saturate(t, -2147483648.0f, 2147483648.0f);
					else if (MODE == I8_FLOAT_I8)
						static_cast<int8_t*>(y)[idx + q] = static_cast<int8_t>(round_saturate(t, -128.0f, 127.0f));
					else
						static_cast<float*>(y)[idx + q] = t;
				}
			}
		}
	};
}

#endif /* AVHIP_CONV_EPILOGUE_HPP_ */
