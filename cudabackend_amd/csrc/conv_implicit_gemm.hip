/*
 * conv_implicit_gemm.hip -- y = act(alpha1 * conv(x, w) + bias + alpha2 * z) + beta * y as an implicit GEMM on MFMA.
 *
 * Replaces the reference's prototype kernel_conv_implicit_gemm / cuda_convolution2dImplicitGemm
 * (src/conv2d_implicit_gemm.cu:150-352), which fixes 3x3 / offset -1 / stride 1 and never finished its weight load.
 * Here the convolution descriptor is honoured: any R x S, signed offsets, stride, dilation, both modes, any padding value.
 *
 * GEMM view: rows = output pixels (n, oh, ow) in NHWC order, columns = output filters, k = (tap, input channel).
 * Both operands are contiguous along the channel part of k, so a 64-byte k-step is a run of channels of one tap:
 *   A chunk = 16 bytes of x[n, ih, iw, c..]   (or the padding value outside the image),
 *   B chunk = 16 bytes of w[k, i, j, c..],
 * fetched straight from global memory (L2 serves the 9-fold tap reuse) into the shared MFMA engine.  Channel counts that
 * are not a multiple of the step are zero-filled in registers, never in HBM.
 * The epilogue is fused into the accumulator store:
 *   floating tensors : fp32 maths, one round-to-nearest-even on store;
 *   int8 -> int32    : exact integer  y = act(sum + bias);
 *   int8 requantised : y = sat_i8(rne(float(sum + bias) * scale[k])), each step a single fp32 rounding;
 *   int8 with float scalars: the header's convention (cast to fp32, scale, cast back with rounding and saturation).
 */
#include "mfma_core.hpp"

namespace
{
	using namespace avhip;

	struct ConvGeom
	{
		int H, W, C, K, R, S, Ho, Wo;
		int pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;
		int flip; /* cross-correlation mode: tap (i, j) reads the input at (R-1-i, S-1-j) */
		int steps_per_tap;
		int64_t pixels; /* N * Ho * Wo */
	};

	template<typename TE>
	struct PixelLoader
	{
		const TE *x;
		const ConvGeom &g;
		TE padv;
		bool vec_ok;
		int ih0[2], iw0[2];
		int64_t img[2]; /* pixel index of (n, 0, 0) */
		bool ok[2];

		__device__ inline PixelLoader(const TE *x_, const ConvGeom &g_, TE padv_, bool vec_ok_, int64_t p0, int frow) :
				x(x_), g(g_), padv(padv_), vec_ok(vec_ok_)
		{
#pragma unroll
			for (int q = 0; q < 2; q++)
			{
				const int64_t p = p0 + frow + 64 * q;
				ok[q] = p < g.pixels;
				const int64_t pp = ok[q] ? p : 0;
				const int ow = static_cast<int>(pp % g.Wo);
				const int oh = static_cast<int>((pp / g.Wo) % g.Ho);
				const int64_t n = pp / (static_cast<int64_t>(g.Wo) * g.Ho);
				ih0[q] = oh * g.stride_h + g.pad_h;
				iw0[q] = ow * g.stride_w + g.pad_w;
				img[q] = n * g.H * g.W;
			}
		}
		__device__ inline uint4 operator()(int step, int q, int part) const
		{
			constexpr int E = 16 / sizeof(TE);
			constexpr int KE = STEP_BYTES / sizeof(TE);
			if (!ok[q])
				return make_uint4(0u, 0u, 0u, 0u);
			const int tap = step / g.steps_per_tap;
			const int c = (step - tap * g.steps_per_tap) * KE + part * E;
			int i = tap / g.S;
			int j = tap - i * g.S;
			if (g.flip)
			{
				i = g.R - 1 - i;
				j = g.S - 1 - j;
			}
			const int ih = ih0[q] + i * g.dil_h;
			const int iw = iw0[q] + j * g.dil_w;
			const int valid = g.C - c;
			if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
				return fetch_chunk<TE>(x + (img[q] + static_cast<int64_t>(ih) * g.W + iw) * g.C + c, valid, vec_ok);
			return splat_chunk<TE>(padv, valid);
		}
	};

	template<typename TE>
	struct FilterLoader
	{
		const TE *w;
		const ConvGeom &g;
		bool vec_ok;
		int k0;
		__device__ inline uint4 operator()(int step, int q, int part) const
		{
			constexpr int E = 16 / sizeof(TE);
			constexpr int KE = STEP_BYTES / sizeof(TE);
			const int k = k0 + (threadIdx.x >> 2) + 64 * q;
			if (k >= g.K)
				return make_uint4(0u, 0u, 0u, 0u);
			const int tap = step / g.steps_per_tap;
			const int c = (step - tap * g.steps_per_tap) * KE + part * E;
			return fetch_chunk<TE>(w + (static_cast<int64_t>(k) * g.R * g.S + tap) * g.C + c, g.C - c, vec_ok);
		}
	};

	__device__ inline int round_saturate(float v, float lo, float hi)
	{
		if (!(v == v))
			return 0;
		float r = rintf(v);
		r = r < lo ? lo : r;
		r = r > hi ? hi : r;
		return static_cast<int>(r);
	}

	/* Floating tensors: TE in, TE out, fp32 bias. */
	template<typename TE>
	__global__ __launch_bounds__(256) void k_conv_igemm_float(const TE *__restrict__ x, const TE *__restrict__ w, const float *__restrict__ bias, const TE *z,
			TE *y, ConvGeom g, TE padv, int vec_ok, float alpha1, float alpha2, float beta, int activation)
	{
		__shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];
		const int64_t p0 = static_cast<int64_t>(blockIdx.x) * BLOCK_M;
		const int k0 = blockIdx.y * BLOCK_N;
		PixelLoader<TE> la(x, g, padv, (vec_ok & 1) != 0, p0, threadIdx.x >> 2);
		FilterLoader<TE> lb { w, g, (vec_ok & 1) != 0, k0 };
		typename Mma<TE>::acc_t acc[2][2];
		block_mma<TE>(lds, g.R * g.S * g.steps_per_tap, la, lb, acc);

		const bool vec_y = (vec_ok & 2) != 0;
		drain_tile<TE>(lds, acc, [&](int r, int col, const float (&v)[4])
		{
			const int64_t p = p0 + r;
			const int k = k0 + col;
			if (p >= g.pixels || k >= g.K)
				return;
			const int valid = g.K - k;
			const int64_t idx = p * g.K + k;
			float t[4];
#pragma unroll
			for (int q = 0; q < 4; q++)
				t[q] = alpha1 * v[q] + ((bias != nullptr && q < valid) ? bias[k + q] : 0.0f);
			if (z != nullptr)
			{
				float zv[4];
				load_vec<TE, 4, float>(z + idx, valid, zv, vec_y);
#pragma unroll
				for (int q = 0; q < 4; q++)
					t[q] += alpha2 * zv[q];
			}
#pragma unroll
			for (int q = 0; q < 4; q++)
				t[q] = activation_forward<float>(activation, t[q]);
			if (beta != 0.0f)
			{
				float yv[4];
				load_vec<TE, 4, float>(y + idx, valid, yv, vec_y);
#pragma unroll
				for (int q = 0; q < 4; q++)
					t[q] += beta * yv[q];
			}
			store_vec<TE, 4, float>(y + idx, valid, t, vec_y);
		});
	}

	enum Int8Epilogue
	{
		I8_EXACT = 0, /* y int32 = act(sum + bias_i32)                                   */
		I8_REQUANT, /* y int8  = sat(rne(float(sum + bias_i32) * scale[k]))             */
		I8_FLOAT_I32, /* float epilogue, y int32                                         */
		I8_FLOAT_I8, /* float epilogue, y int8                                           */
		I8_FLOAT_F32 /* float epilogue, y fp32                                           */
	};

	/* From here on every fp32 operation must round exactly once: the float epilogue on integer sums is specified step by
	 * step (multiply, add, multiply, add), so a*b + c must not be contracted into a fused multiply-add.  The pragma only
	 * governs expressions written below it, which is why the epilogue uses plain operators and no header intrinsics. */
#pragma clang fp contract(off)

	template<int MODE>
	__global__ __launch_bounds__(256) void k_conv_igemm_int8(const int8_t *__restrict__ x, const int8_t *__restrict__ w, const void *__restrict__ bias,
			const void *z, void *y, const float *__restrict__ scale, ConvGeom g, int8_t padv, int vec_ok, float alpha1, float alpha2, float beta, int activation)
	{
		__shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];
		const int64_t p0 = static_cast<int64_t>(blockIdx.x) * BLOCK_M;
		const int k0 = blockIdx.y * BLOCK_N;
		PixelLoader<int8_t> la(x, g, padv, (vec_ok & 1) != 0, p0, threadIdx.x >> 2);
		FilterLoader<int8_t> lb { w, g, (vec_ok & 1) != 0, k0 };
		Mma<int8_t>::acc_t acc[2][2];
		block_mma<int8_t>(lds, g.R * g.S * g.steps_per_tap, la, lb, acc);

		const bool vec_y = (vec_ok & 2) != 0;
		drain_tile<int8_t>(lds, acc, [&](int r, int col, const int (&v)[4])
		{
			const int64_t p = p0 + r;
			const int k = k0 + col;
			if (p >= g.pixels || k >= g.K)
				return;
			const int valid = g.K - k;
			const int64_t idx = p * g.K + k;
			if (MODE == I8_EXACT || MODE == I8_REQUANT)
			{
				int t[4];
#pragma unroll
				for (int q = 0; q < 4; q++)
				{
					t[q] = v[q] + ((bias != nullptr && q < valid) ? static_cast<const int*>(bias)[k + q] : 0);
					if (activation == ACT_RELU && t[q] < 0)
						t[q] = 0;
				}
				if (MODE == I8_EXACT)
				{
					int *dst = static_cast<int*>(y) + idx;
					if (vec_y && valid >= 4)
						*reinterpret_cast<int4*>(dst) = make_int4(t[0], t[1], t[2], t[3]);
					else
					{
#pragma unroll
						for (int q = 0; q < 4; q++)
							if (q < valid)
								dst[q] = t[q];
					}
				}
				else
				{
					int8_t o[4];
#pragma unroll
					for (int q = 0; q < 4; q++)
						o[q] = static_cast<int8_t>(round_saturate(static_cast<float>(t[q]) * (q < valid ? scale[k + q] : 0.0f), -128.0f, 127.0f));
					int8_t *dst = static_cast<int8_t*>(y) + idx;
					if (vec_y && valid >= 4)
						*reinterpret_cast<char4*>(dst) = make_char4(o[0], o[1], o[2], o[3]);
					else
					{
#pragma unroll
						for (int q = 0; q < 4; q++)
							if (q < valid)
								dst[q] = o[q];
					}
				}
			}
			else
			{
#pragma unroll
				for (int q = 0; q < 4; q++)
				{
					if (q >= valid)
						continue;
					float t = alpha1 * static_cast<float>(v[q]);
					if (bias != nullptr)
						t = t + static_cast<const float*>(bias)[k + q];
					if (z != nullptr)
					{
						const float zv = MODE == I8_FLOAT_I32 ? static_cast<float>(static_cast<const int*>(z)[idx + q]) :
											MODE == I8_FLOAT_I8 ? static_cast<float>(static_cast<const int8_t*>(z)[idx + q]) : static_cast<const float*>(z)[idx + q];
						t = t + alpha2 * zv;
					}
					t = activation_forward<float>(activation, t);
					if (beta != 0.0f)
					{
						const float yv = MODE == I8_FLOAT_I32 ? static_cast<float>(static_cast<int*>(y)[idx + q]) :
											MODE == I8_FLOAT_I8 ? static_cast<float>(static_cast<int8_t*>(y)[idx + q]) : static_cast<float*>(y)[idx + q];
						t = t + beta * yv;
					}
					if (MODE == I8_FLOAT_I32)
						static_cast<int*>(y)[idx + q] = round_saturate(t, -2147483648.0f, 2147483520.0f);
					else if (MODE == I8_FLOAT_I8)
						static_cast<int8_t*>(y)[idx + q] = static_cast<int8_t>(round_saturate(t, -128.0f, 127.0f));
					else
						static_cast<float*>(y)[idx + q] = t;
				}
			}
		});
	}

	template<typename TE>
	ConvGeom make_geom(const avhipConvShape &s)
	{
		ConvGeom g;
		g.H = s.H;
		g.W = s.W;
		g.C = s.C;
		g.K = s.K;
		g.R = s.R;
		g.S = s.S;
		g.Ho = s.Ho;
		g.Wo = s.Wo;
		g.pad_h = s.pad_h;
		g.pad_w = s.pad_w;
		g.stride_h = s.stride_h;
		g.stride_w = s.stride_w;
		g.dil_h = s.dil_h;
		g.dil_w = s.dil_w;
		g.flip = (s.mode != 0) ? 1 : 0;
		constexpr int KE = STEP_BYTES / sizeof(TE);
		g.steps_per_tap = (s.C + KE - 1) / KE;
		g.pixels = static_cast<int64_t>(s.N) * s.Ho * s.Wo;
		return g;
	}
	/* bit 0: operand chunks may use 16-byte loads; bit 1: y / z rows may use 4-element vectors of `out_elem` bytes. */
	template<typename TE>
	int vector_flags(const avhipConvShape &s, const void *x, const void *w, const void *y, const void *z, size_t out_elem)
	{
		const bool in_ok = aligned_to(x, 16) && aligned_to(w, 16) && (s.C * sizeof(TE)) % 16 == 0;
		const bool out_ok = s.K % 4 == 0 && aligned_to(y, 4 * out_elem) && (z == nullptr || aligned_to(z, 4 * out_elem));
		return (in_ok ? 1 : 0) | (out_ok ? 2 : 0);
	}

	template<typename TE>
	int launch_float(hipStream_t st, const avhipConvShape &s, const void *x, const void *w, const void *bias, const void *z, void *y, const void *padding_value,
			double alpha1, double alpha2, double beta, int activation)
	{
		const ConvGeom g = make_geom<TE>(s);
		TE padv;
		if (padding_value != nullptr)
			padv = *static_cast<const TE*>(padding_value);
		else
			padv = Traits<TE>::store(0.0f);
		const dim3 grid(ceil_div(g.pixels, BLOCK_M), ceil_div(s.K, BLOCK_N));
		hipLaunchKernelGGL((k_conv_igemm_float<TE>), grid, dim3(256), 0, st, static_cast<const TE*>(x), static_cast<const TE*>(w),
				static_cast<const float*>(bias), static_cast<const TE*>(z), static_cast<TE*>(y), g, padv, vector_flags<TE>(s, x, w, y, z, sizeof(TE)),
				static_cast<float>(alpha1), static_cast<float>(alpha2), static_cast<float>(beta), activation);
		return 0;
	}
	template<int MODE>
	int launch_int8(hipStream_t st, const avhipConvShape &s, const void *x, const void *w, const void *bias, const void *z, void *y, const float *scale,
			const void *padding_value, double alpha1, double alpha2, double beta, int activation)
	{
		const ConvGeom g = make_geom<int8_t>(s);
		const int8_t padv = padding_value != nullptr ? *static_cast<const int8_t*>(padding_value) : static_cast<int8_t>(0);
		const dim3 grid(ceil_div(g.pixels, BLOCK_M), ceil_div(s.K, BLOCK_N));
		hipLaunchKernelGGL((k_conv_igemm_int8<MODE>), grid, dim3(256), 0, st, static_cast<const int8_t*>(x), static_cast<const int8_t*>(w), bias, z, y, scale, g,
				padv, vector_flags<int8_t>(s, x, w, y, z, MODE == I8_REQUANT || MODE == I8_FLOAT_I8 ? 1 : 4), static_cast<float>(alpha1), static_cast<float>(alpha2), static_cast<float>(beta), activation);
		return 0;
	}
}

extern "C" int avhip_conv2d_implicit_gemm(void *stream, int x_dtype, int y_dtype, int bias_dtype, const avhipConvShape *shape, const void *x,
		const void *w, const void *bias, const void *z, void *y, const void *padding_value, double alpha1, double alpha2, double beta, int activation,
		const float *requant_scale)
{
	if (shape == nullptr || x == nullptr || w == nullptr || y == nullptr)
		return AVHIP_BAD_PARAM;
	const avhipConvShape &s = *shape;
	if (s.N <= 0 || s.H <= 0 || s.W <= 0 || s.C <= 0 || s.K <= 0 || s.R <= 0 || s.S <= 0 || s.Ho <= 0 || s.Wo <= 0 || s.stride_h <= 0 || s.stride_w <= 0
			|| s.dil_h <= 0 || s.dil_w <= 0)
		return AVHIP_BAD_PARAM;
	if ((static_cast<int64_t>(s.K) + BLOCK_N - 1) / BLOCK_N > 65535)
		return AVHIP_NOT_SUPPORTED;
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (x_dtype)
	{
		case DT_FLOAT32:
			if (y_dtype != DT_FLOAT32 || requant_scale != nullptr)
				return AVHIP_UNSUPPORTED_DATATYPE;
			return launch_float<float>(st, s, x, w, bias, z, y, padding_value, alpha1, alpha2, beta, activation);
		case DT_FLOAT16:
			if (y_dtype != DT_FLOAT16 || requant_scale != nullptr)
				return AVHIP_UNSUPPORTED_DATATYPE;
			return launch_float<f16_t>(st, s, x, w, bias, z, y, padding_value, alpha1, alpha2, beta, activation);
		case DT_BFLOAT16:
			if (y_dtype != DT_BFLOAT16 || requant_scale != nullptr)
				return AVHIP_UNSUPPORTED_DATATYPE;
			return launch_float<bf16_t>(st, s, x, w, bias, z, y, padding_value, alpha1, alpha2, beta, activation);
		case DT_INT8:
		{
			if (requant_scale != nullptr)
			{
				if (y_dtype != DT_INT8 || (bias != nullptr && bias_dtype != DT_INT32) || z != nullptr
						|| (activation != ACT_LINEAR && activation != ACT_RELU))
					return AVHIP_NOT_SUPPORTED;
				return launch_int8<I8_REQUANT>(st, s, x, w, bias, nullptr, y, requant_scale, padding_value, 1.0, 0.0, 0.0, activation);
			}
			const bool exact = y_dtype == DT_INT32 && (bias == nullptr || bias_dtype == DT_INT32) && z == nullptr && alpha1 == 1.0 && beta == 0.0
					&& (activation == ACT_LINEAR || activation == ACT_RELU);
			if (exact)
				return launch_int8<I8_EXACT>(st, s, x, w, bias, nullptr, y, nullptr, padding_value, 1.0, 0.0, 0.0, activation);
			if (bias != nullptr && bias_dtype != DT_FLOAT32)
				return AVHIP_UNSUPPORTED_DATATYPE;
			switch (y_dtype)
			{
				case DT_INT32:
					return launch_int8<I8_FLOAT_I32>(st, s, x, w, bias, z, y, nullptr, padding_value, alpha1, alpha2, beta, activation);
				case DT_INT8:
					return launch_int8<I8_FLOAT_I8>(st, s, x, w, bias, z, y, nullptr, padding_value, alpha1, alpha2, beta, activation);
				case DT_FLOAT32:
					return launch_int8<I8_FLOAT_F32>(st, s, x, w, bias, z, y, nullptr, padding_value, alpha1, alpha2, beta, activation);
				default:
					return AVHIP_UNSUPPORTED_DATATYPE;
			}
		}
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}
