/*
 * conv_implicit_gemm.hip -- y = act(alpha1 * conv(x, w) + bias + alpha2 * z) + beta * y as an implicit GEMM on MFMA.
 *
 * Replaces the reference's prototype kernel_conv_implicit_gemm / cuda_convolution2dImplicitGemm
 * (src/conv2d_implicit_gemm.cu:150-352), which fixes 3x3 / offset -1 / stride 1 and never finished its weight load.
 * Here the convolution descriptor is honoured: any R x S, signed offsets, stride, dilation, both modes, any padding value.
 *
 * GEMM view: rows = output pixels (n, oh, ow) in NHWC order, columns = output filters, k = (tap, input channel).
 * Both operands are contiguous along the channel part of k, so a 128-byte k-step is a run of channels of one tap:
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
#include <algorithm>
#include <cstring>
#include <type_traits>

#include "conv_epilogue.hpp"
#include "conv_pointwise.hpp"
#include "conv_small.hpp"
#include "conv_stem.hpp"
#include "conv_thin.hpp"
#include "conv_tile.hpp"
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
		int64_t images; /* N */
	};

	/* Walks k = (tap, channel slice) in order; shared by both operand loaders. */
	struct TapCursor
	{
		int i = 0, j = 0, slice = 0, tap = 0;
		/* to k-step `step` of the walk */
		__device__ inline void seek(const ConvGeom &g, int step)
		{
			tap = step / g.steps_per_tap;
			slice = step - tap * g.steps_per_tap;
			i = tap / g.S;
			j = tap - i * g.S;
		}
		__device__ inline void advance(const ConvGeom &g)
		{
			if (++slice == g.steps_per_tap)
			{
				slice = 0;
				tap++;
				if (++j == g.S)
				{
					j = 0;
					i++;
				}
			}
		}
	};

	/* Bit t = i * S + j of the result: tap (i, j) of the window whose origin is (ih0, iw0) reads a pixel inside the image.
	 * Rows and columns are tested separately (R + S tests, no division) and combined. */
	__device__ inline unsigned int inside_mask(const ConvGeom &g, int ih0, int iw0)
	{
		unsigned int columns = 0, m = 0;
		for (int j = 0; j < g.S; j++)
		{
			const int iw = iw0 + (g.flip ? g.S - 1 - j : j) * g.dil_w;
			if (iw >= 0 && iw < g.W)
				columns |= 1u << j;
		}
		for (int i = 0; i < g.R; i++)
		{
			const int ih = ih0 + (g.flip ? g.R - 1 - i : i) * g.dil_h;
			if (ih >= 0 && ih < g.H)
				m |= columns << (i * g.S);
		}
		return m;
	}

	/* Rows of A are output pixels; a chunk is 16 bytes of channels of the input pixel that tap (i, j) reads.
	 * General form: any alignment, any channel count, any padding value. */
	template<typename TE, bool FAST>
	struct PixelLoader
	{
		const TE *x;
		const ConvGeom &g;
		TE padv;
		bool vec_ok;
		TapCursor cur;
		int ih0[FETCH_PASSES], iw0[FETCH_PASSES];
		int64_t img[FETCH_PASSES]; /* pixel index of (n, 0, 0) */
		bool ok[FETCH_PASSES];

		__device__ inline PixelLoader(const TE *x_, const ConvGeom &g_, TE padv_, bool vec_ok_, int64_t p0) :
				x(x_), g(g_), padv(padv_), vec_ok(vec_ok_)
		{
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int64_t p = p0 + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
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
		__device__ inline uint4 load(int q, int part) const
		{
			constexpr int E = 16 / sizeof(TE);
			constexpr int KE = STEP_BYTES / sizeof(TE);
			if (!ok[q] || cur.i >= g.R)
				return make_uint4(0u, 0u, 0u, 0u);
			const int c = cur.slice * KE + part * E;
			const int i = g.flip ? g.R - 1 - cur.i : cur.i;
			const int j = g.flip ? g.S - 1 - cur.j : cur.j;
			const int ih = ih0[q] + i * g.dil_h;
			const int iw = iw0[q] + j * g.dil_w;
			const int valid = g.C - c;
			if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
				return fetch_chunk<TE>(x + (img[q] + static_cast<int64_t>(ih) * g.W + iw) * g.C + c, valid, vec_ok);
			return splat_chunk<TE>(padv, valid);
		}
		__device__ inline void next()
		{
			cur.advance(g);
		}
	};
	/*
	 * Fast form: x 16-byte aligned and below 2 GiB, C a multiple of the chunk, zero padding value, at most 32 taps.
	 * Everything that depends on the output pixel is computed once per work-item: the byte offset of the window origin
	 * (with this work-item's chunk already added) and a bit mask of the taps that fall inside the image.  Everything that
	 * depends on the k-slice is uniform and lives in scalar registers.  A chunk then costs one add, one bit test and one
	 * select before its branch-free buffer load, whose offset is OUT_OF_RANGE (hardware returns zeros) when it does not exist.
	 */
	template<typename TE>
	struct PixelLoader<TE, true>
	{
		__amdgpu_buffer_rsrc_t rsrc;
		const ConvGeom &g;
		TapCursor cur;
		unsigned int origin[FETCH_PASSES]; /* byte offset of (n, ih0, iw0, chunk channel); may wrap below zero, never used then */
		unsigned int inside[FETCH_PASSES]; /* bit t: tap t reads a pixel inside the image */
		int chunk_channel; /* first channel of this work-item's chunk within a k-slice */
		unsigned int tap_bytes; /* uniform: offset of the current tap and slice relative to the window origin */

		__device__ inline PixelLoader(const TE *x, const ConvGeom &g_, TE, bool, int64_t p0) :
				g(g_)
		{
			constexpr int E = 16 / sizeof(TE);
			rsrc = make_buffer(x, static_cast<unsigned int>(g.images * g.H * g.W * g.C * sizeof(TE)));
			chunk_channel = (threadIdx.x % STEP_CHUNKS) * E;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				/* the tensor is below 2 GiB, so pixel indices fit 32 bits and the divisions stay cheap */
				const unsigned int p = static_cast<unsigned int>(p0) + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
				const bool ok = p < static_cast<unsigned int>(g.pixels);
				const unsigned int pp = ok ? p : 0u;
				const unsigned int row = pp / static_cast<unsigned int>(g.Wo);
				const int ow = static_cast<int>(pp - row * g.Wo);
				const unsigned int n = row / static_cast<unsigned int>(g.Ho);
				const int oh = static_cast<int>(row - n * g.Ho);
				const int ih0 = oh * g.stride_h + g.pad_h;
				const int iw0 = ow * g.stride_w + g.pad_w;
				origin[q] = static_cast<unsigned int>((static_cast<int>(n * g.H + ih0) * g.W + iw0) * g.C + chunk_channel) * static_cast<unsigned int>(sizeof(TE));
				inside[q] = ok ? inside_mask(g, ih0, iw0) : 0u;
			}
			set_tap();
		}
		__device__ inline void set_tap()
		{
			const int i = g.flip ? g.R - 1 - cur.i : cur.i;
			const int j = g.flip ? g.S - 1 - cur.j : cur.j;
			tap_bytes = static_cast<unsigned int>(((i * g.dil_h) * g.W + j * g.dil_w) * g.C) * static_cast<unsigned int>(sizeof(TE))
					+ static_cast<unsigned int>(cur.slice) * STEP_BYTES;
		}
		__device__ inline uint4 load(int q, int) const
		{
			constexpr int KE = STEP_BYTES / sizeof(TE);
			const bool exists = (((inside[q] >> cur.tap) & 1u) != 0u) & (cur.slice * KE + chunk_channel < g.C) & (cur.tap < 32);
			return buffer_fetch(rsrc, exists ? origin[q] + tap_bytes : OUT_OF_RANGE);
		}
		__device__ inline void next()
		{
			cur.advance(g);
			set_tap();
		}
		__device__ inline void seek(int step)
		{
			cur.seek(g, step);
			set_tap();
		}
	};

	/* Rows of B are output filters; a chunk is 16 bytes of channels of w[k, i, j, :]. */
	template<typename TE, bool FAST>
	struct FilterLoader
	{
		const ConvGeom &g;
		bool vec_ok;
		TapCursor cur;
		const TE *rows[FETCH_PASSES];
		__device__ inline FilterLoader(const TE *w, const ConvGeom &g_, bool vec_ok_, int k0) :
				g(g_), vec_ok(vec_ok_)
		{
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int k = k0 + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
				rows[q] = k < g.K ? w + static_cast<int64_t>(k) * g.R * g.S * g.C : nullptr;
			}
		}
		__device__ inline uint4 load(int q, int part) const
		{
			constexpr int E = 16 / sizeof(TE);
			constexpr int KE = STEP_BYTES / sizeof(TE);
			if (rows[q] == nullptr || cur.i >= g.R)
				return make_uint4(0u, 0u, 0u, 0u);
			const int c = cur.slice * KE + part * E;
			return fetch_chunk<TE>(rows[q] + static_cast<int64_t>(cur.tap) * g.C + c, g.C - c, vec_ok);
		}
		__device__ inline void next()
		{
			cur.advance(g);
		}
	};
	template<typename TE>
	struct FilterLoader<TE, true>
	{
		__amdgpu_buffer_rsrc_t rsrc;
		const ConvGeom &g;
		TapCursor cur;
		unsigned int origin[FETCH_PASSES]; /* byte offset of w[k, 0, 0, chunk channel]; OUT_OF_RANGE for k >= K stays out of range */
		int chunk_channel;
		__device__ inline FilterLoader(const TE *w, const ConvGeom &g_, bool, int k0) :
				g(g_)
		{
			constexpr int E = 16 / sizeof(TE);
			rsrc = make_buffer(w, static_cast<unsigned int>(static_cast<int64_t>(g.K) * g.R * g.S * g.C * sizeof(TE)));
			chunk_channel = (threadIdx.x % STEP_CHUNKS) * E;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int k = k0 + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
				origin[q] = k < g.K ? static_cast<unsigned int>((k * g.R * g.S * g.C + chunk_channel) * sizeof(TE)) : OUT_OF_RANGE;
			}
		}
		__device__ inline uint4 load(int q, int) const
		{
			constexpr int KE = STEP_BYTES / sizeof(TE);
			const unsigned int tap_bytes = static_cast<unsigned int>(cur.tap * g.C) * static_cast<unsigned int>(sizeof(TE))
					+ static_cast<unsigned int>(cur.slice) * STEP_BYTES;
			const bool exists = (cur.slice * KE + chunk_channel < g.C) & (cur.i < g.R);
			return buffer_fetch(rsrc, exists ? origin[q] + tap_bytes : OUT_OF_RANGE);
		}
		__device__ inline void next()
		{
			cur.advance(g);
		}
		__device__ inline void seek(int step)
		{
			cur.seek(g, step);
		}
	};

	/*
	 * Few input channels (a network's first layer: 3 or 4 planes): one tap holds far less than a 128-byte k-step, so k is
	 * taken as the flattened (tap, channel) index of the filter row, R*S*C elements long, and a 16-byte chunk is gathered
	 * from 16 / PB pieces of PB bytes, each from the tap it falls into.  PB is the largest power of two (2..16) that divides
	 * the bytes of one pixel, so a piece never straddles two taps.  Which tap a piece belongs to does not depend on the
	 * output pixel: it is worked out once per k-step; per pixel there is the window origin and the inside-mask as in the
	 * fast loader.  Same preconditions as the fast loader (zero padding value, 32-bit offsets, at most 32 taps).
	 */
	template<int PB> struct Piece;
	template<> struct Piece<16>
	{
		typedef u32x4_t type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(off), 0, 0);
		}
	};
	template<> struct Piece<8>
	{
		typedef __attribute__((__vector_size__(2 * sizeof(unsigned int)))) unsigned int type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b64(r, static_cast<int>(off), 0, 0);
		}
	};
	template<> struct Piece<4>
	{
		typedef unsigned int type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b32(r, static_cast<int>(off), 0, 0);
		}
	};
	template<> struct Piece<2>
	{
		typedef unsigned short type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b16(r, static_cast<int>(off), 0, 0);
		}
	};
	template<int PB>
	union PieceChunk
	{
		uint4 u;
		typename Piece<PB>::type piece[16 / PB];
	};

	template<typename TE, int PB>
	struct PackedPixelLoader
	{
		static constexpr int NP = 16 / PB;
		__amdgpu_buffer_rsrc_t rsrc;
		const ConvGeom &g;
		unsigned int origin[FETCH_PASSES]; /* byte offset of (n, ih0, iw0, 0) */
		unsigned int inside[FETCH_PASSES]; /* bit t: tap t reads a pixel inside the image */
		unsigned int rel[NP]; /* byte offset of each piece of the current k-step relative to the window origin */
		unsigned int bit[NP]; /* the piece's tap as a mask bit; 0 when the piece lies past the end of k */
		unsigned int k_byte; /* flattened-k byte position of this work-item's chunk in the current step */

		__device__ inline PackedPixelLoader(const TE *x, const ConvGeom &g_, int64_t p0) :
				g(g_)
		{
			rsrc = make_buffer(x, static_cast<unsigned int>(g.images * g.H * g.W * g.C * sizeof(TE)));
			const unsigned int CB = g.C * sizeof(TE);
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const unsigned int p = static_cast<unsigned int>(p0) + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
				const bool ok = p < static_cast<unsigned int>(g.pixels);
				const unsigned int pp = ok ? p : 0u;
				const unsigned int row = pp / static_cast<unsigned int>(g.Wo);
				const int ow = static_cast<int>(pp - row * g.Wo);
				const unsigned int n = row / static_cast<unsigned int>(g.Ho);
				const int oh = static_cast<int>(row - n * g.Ho);
				const int ih0 = oh * g.stride_h + g.pad_h;
				const int iw0 = ow * g.stride_w + g.pad_w;
				origin[q] = static_cast<unsigned int>((static_cast<int>(n * g.H + ih0) * g.W + iw0)) * CB;
				inside[q] = ok ? inside_mask(g, ih0, iw0) : 0u;
			}
			k_byte = (threadIdx.x % STEP_CHUNKS) * 16;
			place();
		}
		__device__ inline void place()
		{
			const unsigned int CB = g.C * sizeof(TE);
			const unsigned int k_bytes = g.R * g.S * CB;
#pragma unroll
			for (int e = 0; e < NP; e++)
			{
				const unsigned int b = k_byte + e * PB;
				const unsigned int tap = b / CB;
				const unsigned int within = b - tap * CB;
				int i = tap / g.S, j = tap - (tap / g.S) * g.S;
				if (g.flip)
				{
					i = g.R - 1 - i;
					j = g.S - 1 - j;
				}
				rel[e] = static_cast<unsigned int>((i * g.dil_h) * g.W + j * g.dil_w) * CB + within;
				bit[e] = b < k_bytes ? 1u << (tap & 31u) : 0u;
			}
		}
		__device__ inline uint4 load(int q, int) const
		{
			PieceChunk<PB> c;
#pragma unroll
			for (int e = 0; e < NP; e++)
				c.piece[e] = Piece<PB>::get(rsrc, (inside[q] & bit[e]) != 0u ? origin[q] + rel[e] : OUT_OF_RANGE);
			return c.u;
		}
		__device__ inline void next()
		{
			k_byte += STEP_BYTES;
			place();
		}
	};
	template<typename TE, int PB>
	struct PackedFilterLoader
	{
		static constexpr int NP = 16 / PB;
		__amdgpu_buffer_rsrc_t rsrc;
		unsigned int origin[FETCH_PASSES]; /* byte offset of row k of w; OUT_OF_RANGE for k >= K */
		unsigned int k_byte, k_bytes;
		__device__ inline PackedFilterLoader(const TE *w, const ConvGeom &g, int k0)
		{
			k_bytes = g.R * g.S * g.C * sizeof(TE);
			rsrc = make_buffer(w, static_cast<unsigned int>(g.K) * k_bytes);
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int k = k0 + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
				origin[q] = k < g.K ? static_cast<unsigned int>(k) * k_bytes : OUT_OF_RANGE;
			}
			k_byte = (threadIdx.x % STEP_CHUNKS) * 16;
		}
		__device__ inline uint4 load(int q, int) const
		{
			PieceChunk<PB> c;
#pragma unroll
			for (int e = 0; e < NP; e++)
				c.piece[e] = Piece<PB>::get(rsrc, k_byte + e * PB < k_bytes ? origin[q] + k_byte + e * PB : OUT_OF_RANGE);
			return c.u;
		}
		__device__ inline void next()
		{
			k_byte += STEP_BYTES;
		}
	};

	/* One kernel for every epilogue: Epi is FloatEpilogue<TE> or Int8Epilogue<mode>.  FAST instances use the branch-free
	 * loaders and are launched for LINEAR / RELU only; everything else runs the general instance.  A FAST instance without
	 * VEC is for filter counts that are not a multiple of four (21 classes, 255 = 3 x 85 box values) or unaligned y, a FAST
	 * instance with ACT_ANY for the seven other activations: the loaders are what makes the general instance slow, not its
	 * element-wise stores or its switch over the activations (a 3x3 layer with a sigmoid: 139 us there). */
	template<typename TE, bool FAST, typename Epi, bool VEC = FAST, int ACT = (FAST ? ACT_SIMPLE : ACT_ANY)>
	__global__ __launch_bounds__(256, 2) void k_conv_igemm(const TE *__restrict__ x, const TE *__restrict__ w, ConvGeom g, TE padv, int vec_ok, Epi epi)
	{
		__shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];
		/* neighbouring pixel blocks read overlapping input windows and the filter blocks of a pixel block read the same ones:
		 * one XCD (one L2) gets a contiguous run of them */
		unsigned int pixel_block, filter_block;
		xcd_tile(pixel_block, filter_block);
		const int64_t p0 = static_cast<int64_t>(pixel_block) * BLOCK_M;
		const int k = filter_block * BLOCK_N + drain_column<2>();
		typename Epi::Columns columns;
		epi.load_columns(k, columns); /* issued before the k loop: its latency is hidden behind the whole convolution */

		PixelLoader<TE, FAST> la(x, g, padv, (vec_ok & 1) != 0, p0);
		FilterLoader<TE, FAST> lb(w, g, (vec_ok & 1) != 0, filter_block * BLOCK_N);
		typename Mma<TE>::acc_t acc[2][2];
		block_mma<TE>(lds, g.R * g.S * g.steps_per_tap, la, lb, acc);

		auto row_out = [&](int r, const typename Epi::scalar_t (&v)[4], int) __attribute__((always_inline))
		{
			const int64_t p = p0 + r;
			if (p < g.pixels && k < g.K)
				epi.template store<ACT, VEC>(p, k, v, columns); /* VEC instances store whole 4-filter vectors */
		};
		/* (the nine-way switch of ACT_ANY, once per row of a fully unrolled hand-over, was too much to unroll: the accumulators
		 * then lived in scratch memory and a layer with a sigmoid took 139 us against 12 us with ReLU) */
		if constexpr (ACT == ACT_ANY)
			drain_tile_rolled<TE, 2, 2>(lds, acc, row_out);
		else
			drain_tile<TE, 2, 2>(lds, acc, row_out);
	}

	template<typename TE, int PB, typename Epi>
	__global__ __launch_bounds__(256, 2) void k_conv_igemm_packed(const TE *__restrict__ x, const TE *__restrict__ w, ConvGeom g, Epi epi)
	{
		__shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];
		/* neighbouring pixel blocks read overlapping input windows and the filter blocks of a pixel block read the same ones:
		 * one XCD (one L2) gets a contiguous run of them */
		unsigned int pixel_block, filter_block;
		xcd_tile(pixel_block, filter_block);
		const int64_t p0 = static_cast<int64_t>(pixel_block) * BLOCK_M;
		const int k = filter_block * BLOCK_N + drain_column<2>();
		typename Epi::Columns columns;
		epi.load_columns(k, columns);

		PackedPixelLoader<TE, PB> la(x, g, p0);
		PackedFilterLoader<TE, PB> lb(w, g, filter_block * BLOCK_N);
		typename Mma<TE>::acc_t acc[2][2];
		block_mma<TE>(lds, (g.R * g.S * g.C * static_cast<int>(sizeof(TE)) + STEP_BYTES - 1) / STEP_BYTES, la, lb, acc);

		drain_tile<TE, 2, 2>(lds, acc, [&](int r, const typename Epi::scalar_t (&v)[4], int) __attribute__((always_inline))
		{
			const int64_t p = p0 + r;
			if (p < g.pixels && k < g.K)
				epi.template store<ACT_SIMPLE, true>(p, k, v, columns);
		});
	}

	/*
	 * Split k: for layers with few output pixels and a long k (the last stages of a deep network at a small batch) the
	 * 128 x 128 tiling yields a few dozen workgroups, each walking thousands of k elements alone.  Here blockIdx.z takes an
	 * even number of k-steps of the walk and stores the raw fp32 sums of its part to partial[z][pixel][filter]; k_split_reduce
	 * adds the parts and applies the epilogue.  Branch-free loaders only (aligned chunks, zero padding value).
	 */
	template<typename TE>
	__global__ __launch_bounds__(256, 2) void k_conv_igemm_split(const TE *__restrict__ x, const TE *__restrict__ w, ConvGeom g, int steps_per_split,
			float *__restrict__ partial)
	{
		__shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];
		unsigned int pixel_block, filter_block;
		xcd_tile(pixel_block, filter_block);
		const int64_t p0 = static_cast<int64_t>(pixel_block) * BLOCK_M;
		const int k = filter_block * BLOCK_N + drain_column<2>();
		const int total = g.R * g.S * g.steps_per_tap, first = static_cast<int>(blockIdx.z) * steps_per_split;
		const int steps = total - first < steps_per_split ? total - first : steps_per_split;

		const TE no_padding_value = TE();
		PixelLoader<TE, true> la(x, g, no_padding_value, true, p0);
		FilterLoader<TE, true> lb(w, g, true, filter_block * BLOCK_N);
		la.seek(first);
		lb.seek(first);
		typename Mma<TE>::acc_t acc[2][2];
		block_mma<TE>(lds, steps, la, lb, acc);

		float *part = partial + static_cast<int64_t>(blockIdx.z) * g.pixels * g.K;
		drain_tile<TE, 2, 2>(lds, acc, [&](int r, const float (&v)[4], int) __attribute__((always_inline))
		{
			const int64_t p = p0 + r;
			if (p < g.pixels && k < g.K)
			{
				typedef float f32x4 __attribute__((ext_vector_type(4)));
				const f32x4 sums = { v[0], v[1], v[2], v[3] };
				*reinterpret_cast<f32x4*>(part + p * g.K + k) = sums;
			}
		});
	}
	/* y = epilogue(sum over the parts), four filters of a pixel per work-item */
	template<typename TE>
	__global__ __launch_bounds__(256) void k_split_reduce(const float *__restrict__ partial, int splits, int64_t plane, FloatEpilogue<TE> epi)
	{
		const int64_t e = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
		if (e >= plane)
			return;
		typedef float f32x4 __attribute__((ext_vector_type(4)));
		/* four parts at a time, so that their loads are in flight together; the sum runs in the order of the parts either way */
		f32x4 sum = *reinterpret_cast<const f32x4*>(partial + e);
		int z = 1;
		for (; z + 4 <= splits; z += 4)
		{
			f32x4 part[4];
#pragma unroll
			for (int u = 0; u < 4; u++)
				part[u] = *reinterpret_cast<const f32x4*>(partial + (z + u) * plane + e);
#pragma unroll
			for (int u = 0; u < 4; u++)
				sum += part[u];
		}
		for (; z < splits; z++)
			sum += *reinterpret_cast<const f32x4*>(partial + z * plane + e);
		const int k = static_cast<int>(e % epi.K);
		typename FloatEpilogue<TE>::Columns columns;
		epi.load_columns(k, columns);
		const float v[4] = { sum[0], sum[1], sum[2], sum[3] };
		epi.template store_at<ACT_ANY, false, 4>(e, k, v, columns);
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
		g.images = s.N;
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

	/* The branch-free loaders need aligned, complete chunks (bit 0 of flags), a zero padding value and 32-bit byte offsets. */
	template<typename TE>
	bool fast_path_ok(const avhipConvShape &s, int flags, const void *padding_value, bool tap_mask = true)
	{
		bool zero_padding = true;
		if (padding_value != nullptr)
			for (size_t i = 0; i < sizeof(TE); i++)
				zero_padding = zero_padding && static_cast<const unsigned char*>(padding_value)[i] == 0;
		const int64_t x_bytes = static_cast<int64_t>(s.N) * s.H * s.W * s.C * sizeof(TE);
		const int64_t w_bytes = static_cast<int64_t>(s.K) * s.R * s.S * s.C * sizeof(TE);
		const int64_t pixels = static_cast<int64_t>(s.N) * s.Ho * s.Wo;
		return (flags & 1) != 0 && zero_padding && x_bytes < (1ll << 31) && w_bytes < (1ll << 31) && pixels < (1ll << 31) - BLOCK_M
				&& (!tap_mask || s.R * s.S <= 32); /* the gather kernel keeps one bit per tap: which taps of a pixel lie inside the image */
	}

	template<typename TE, typename Epi>
	int launch(hipStream_t st, const avhipConvShape &s, const void *x, const void *w, const void *padding_value, int flags, const Epi &epi)
	{
		/* (the integer epilogues are only ever asked for LINEAR and RELU) */
		constexpr bool integer_epilogue = std::is_same<Epi, Int8Epilogue<I8_EXACT>>::value || std::is_same<Epi, Int8Epilogue<I8_REQUANT>>::value;
		constexpr int GENERAL_ACT = integer_epilogue ? ACT_SIMPLE : ACT_ANY;
		const ConvGeom g = make_geom<TE>(s);
		TE padv;
		if (padding_value != nullptr)
			padv = *static_cast<const TE*>(padding_value);
		else
			std::memset(&padv, 0, sizeof(TE));
		const dim3 grid(ceil_div(g.pixels, BLOCK_M), ceil_div(s.K, BLOCK_N));
		/* the branch-free instances also store whole 4-filter vectors (streaming stores): K % 4 == 0 and y, z aligned (bit 1) */
		const bool fast = fast_path_ok<TE>(s, flags, padding_value) && is_simple_activation(epi.activation) && (flags & 2) != 0;
		/* few input channels: pack (tap, channel) into the k-steps instead of spending a step per tap.  Below 64 bytes per pixel:
		 * at 64 (half a k-step per tap) the kernels below are the faster ones, measured on 3x3 layers of 64 int8 / 32 bf16 / 16 fp32
		 * channels (12 against 28 us, 21 against 52 us, 82 against 113 us); at 48 and 32 bytes these are (16 against 22 us, 13 against 22 us) */
		const int pixel_bytes = s.C * static_cast<int>(sizeof(TE));
		if (pixel_bytes < STEP_BYTES / 2 && s.R * s.S > 1 && fast_path_ok<TE>(s, 1, padding_value, false) && is_simple_activation(epi.activation)
				&& (flags & 2) != 0)
		{
			/* a pixel of exactly 8 bytes and a small filter: operands straight into registers, no k loop */
			if (conv_stem_launch<TE, Epi>(st, s, x, w, epi))
				return 0;
			/* the image tile in LDS, the operand gathered from there: filters of any number of taps */
			if (conv_thin_launch<TE, Epi>(st, s, x, w, epi))
				return 0;
			int pb = 16;
			while (pb > 1 && (pixel_bytes % pb != 0 || !aligned_to(x, pb) || !aligned_to(w, pb)))
				pb /= 2;
			pb = (pb < static_cast<int>(sizeof(TE)) || s.R * s.S > 32) ? 0 : pb; /* the gather kernel's tap mask has 32 bits */
#define AVHIP_PACKED(PB) hipLaunchKernelGGL((k_conv_igemm_packed<TE, PB, Epi>), grid, dim3(256), 0, st, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi)
			switch (pb)
			{
				case 16:
					AVHIP_PACKED(16);
					return 0;
				case 8:
					AVHIP_PACKED(8);
					return 0;
				case 4:
					AVHIP_PACKED(4);
					return 0;
				case 2:
					AVHIP_PACKED(2);
					return 0;
				default:
					break;
			}
#undef AVHIP_PACKED
		}
		/* a problem of a few big tiles goes to the kernel with one 32 x 32 tile per wavefront */
		if (fast && conv_small_launch<TE, Epi>(st, s, x, w, epi, static_cast<int64_t>(grid.x) * grid.y))
			return 0;
		/* one-tap filters are plain matrix products with a short k: a persistent kernel pipelines across tiles */
		if (fast && s.R * s.S == 1 && conv_pointwise_launch<TE, Epi>(st, s, x, w, epi))
			return 0;
		/* stride-1 filters with more than one tap first try the kernel that keeps an image tile resident in LDS */
		/* (that kernel has no limit on the number of taps) */
		const bool fast_tile = fast || (fast_path_ok<TE>(s, flags, padding_value, false) && is_simple_activation(epi.activation) && (flags & 2) != 0);
		if (fast_tile && s.R * s.S > 1 && conv_tile_launch<TE, Epi>(st, s, x, w, epi))
			return 0;
		if (fast)
			hipLaunchKernelGGL((k_conv_igemm<TE, true, Epi>), grid, dim3(256), 0, st, static_cast<const TE*>(x), static_cast<const TE*>(w), g, padv, flags, epi);
		else if (fast_path_ok<TE>(s, flags, padding_value))
		{
			/* the branch-free loaders with what the layer needs of the general epilogue */
			const bool vec = (flags & 2) != 0;
#define AVHIP_GATHER(VEC, ACT) hipLaunchKernelGGL((k_conv_igemm<TE, true, Epi, VEC, ACT>), grid, dim3(256), 0, st, static_cast<const TE*>(x), \
		static_cast<const TE*>(w), g, padv, flags, epi)
			if (is_simple_activation(epi.activation))
				AVHIP_GATHER(false, ACT_SIMPLE);
			else if (vec && !integer_epilogue)
			{
				if constexpr (!integer_epilogue)
					AVHIP_GATHER(true, ACT_ANY);
			}
			else /* both at once is left to the general instance */
				hipLaunchKernelGGL((k_conv_igemm<TE, false, Epi, false, GENERAL_ACT>), grid, dim3(256), 0, st, static_cast<const TE*>(x), static_cast<const TE*>(w), g, padv, flags, epi);
#undef AVHIP_GATHER
		}
		else
			hipLaunchKernelGGL((k_conv_igemm<TE, false, Epi, false, GENERAL_ACT>), grid, dim3(256), 0, st, static_cast<const TE*>(x), static_cast<const TE*>(w), g, padv, flags, epi);
		return 0;
	}
	template<typename TE>
	int launch_float(hipStream_t st, const avhipConvShape &s, const void *x, const void *w, const void *bias, const void *z, void *y, const void *padding_value,
			double alpha1, double alpha2, double beta, int activation)
	{
		const int flags = vector_flags<TE>(s, x, w, y, z, sizeof(TE));
		const FloatEpilogue<TE> epi { static_cast<const float*>(bias), static_cast<const TE*>(z), static_cast<TE*>(y), static_cast<float>(alpha1),
				static_cast<float>(alpha2), static_cast<float>(beta), activation, s.K, (flags & 2) != 0 };
		return launch<TE>(st, s, x, w, padding_value, flags, epi);
	}
	template<int MODE>
	int launch_int8(hipStream_t st, const avhipConvShape &s, const void *x, const void *w, const void *bias, const void *z, void *y, const float *scale,
			const void *padding_value, double alpha1, double alpha2, double beta, int activation)
	{
		const int flags = vector_flags<int8_t>(s, x, w, y, z, MODE == I8_REQUANT || MODE == I8_FLOAT_I8 ? 1 : 4);
		const Int8Epilogue<MODE> epi { bias, z, y, scale, static_cast<float>(alpha1), static_cast<float>(alpha2), static_cast<float>(beta), activation, s.K,
				(flags & 2) != 0 };
		return launch<int8_t>(st, s, x, w, padding_value, flags, epi);
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

namespace
{
	/* Whether to split k, into how many parts of how many steps, and the workspace that takes: worth it when the plain tiling
	 * leaves most compute units idle for a long walk.  Estimates in microseconds (fitted to layers of 196 to 6272 pixels with
	 * 1024 to 4608 elements of k): 4 + 0.7 per k-step for a workgroup of the plain gather kernel (less in the image-tile kernel); for the split, 10 for the two
	 * launches and their prologues, 0.7 per step of a part, 0.25 per part and the parts read back at 4 TB/s in the reduction;
	 * the one-wavefront-per-tile kernel by its own estimate where the launcher would use it. */
	struct SplitPlan
	{
		int splits, steps_per_split;
		int64_t bytes;
	};
	template<typename TE>
	bool split_k_plan(const avhipConvShape &s, SplitPlan &plan)
	{
		constexpr int KE = STEP_BYTES / sizeof(TE);
		const int64_t pixels = static_cast<int64_t>(s.N) * s.Ho * s.Wo;
		const int64_t tiles = ((pixels + BLOCK_M - 1) / BLOCK_M) * ((static_cast<int64_t>(s.K) + BLOCK_N - 1) / BLOCK_N);
		const int64_t steps = static_cast<int64_t>(s.R) * s.S * ((s.C + KE - 1) / KE);
		/* the branch-free loaders: whole 16-byte chunks of channels, one mask bit per tap */
		if (tiles >= 256 || steps < 8 || steps > (1 << 20) || (s.C * sizeof(TE)) % 16 != 0 || s.R * s.S > 32)
			return false;
		int64_t parts = std::min<int64_t>(512 / tiles, steps / 4);
		if (parts < 2)
			return false;
		const int64_t per_part = ((steps + parts - 1) / parts + 1) / 2 * 2; /* even: the engine runs its steps in pairs */
		parts = (steps + per_part - 1) / per_part;
		if (parts < 2 || parts > 65535)
			return false;
		const double plane_bytes = static_cast<double>(pixels) * s.K * 4.0;
		double other = 4.0 + 0.7 * static_cast<double>(steps);
		int64_t plain_workgroups = tiles;
		if (s.stride_h == 1 && s.stride_w == 1 && s.dil_h == 1 && s.dil_w == 1 && s.R * s.S > 1 && s.Ho * s.Wo >= 128)
		{
			/* the image-tile kernel takes such layers: 0.47 us per step for a workgroup with a compute unit to itself, 0.68 us
			 * when two share one, 3.6 us around the loop */
			const int64_t workgroups = static_cast<int64_t>(s.N) * ((s.K + 63) / 64) * ((s.Ho * s.Wo + 255) / 256);
			other = 3.6 + (workgroups <= 256 ? 0.47 : 0.68) * static_cast<double>(steps);
			plain_workgroups = workgroups;
		}
		/* neither path is faster than the matrix cores of the compute units it occupies (what decides for fp32, whose MFMAs
		 * take eight times as long per element): flops per microsecond of the chip as sustained on random data */
		const double chip = sizeof(TE) == 4 ? 1.55e8 : 1.87e9;
		const double flops = 2.0 * static_cast<double>(pixels) * s.K * s.C * s.R * s.S;
		other = std::max(other, flops / (chip * std::min(1.0, static_cast<double>(plain_workgroups) / 256.0)));
		if (s.R * s.S <= 32 && conv_small_preferred(s, static_cast<int>(sizeof(TE)), tiles))
		{
			const double wavefronts = static_cast<double>(((pixels + 31) / 32) * ((s.K + 31) / 32));
			const double small = std::max(conv_small_estimate(s, static_cast<int>(sizeof(TE)), tiles).small_us, flops / (chip * std::min(1.0, wavefronts / 1024.0)));
			other = std::min(other, small);
		}
		const double walk = std::max(0.7 * static_cast<double>(per_part), flops / (chip * std::min(1.0, static_cast<double>(tiles * parts) / 256.0)));
		const double split = 10.0 + walk + 0.25 * static_cast<double>(parts) + plane_bytes * static_cast<double>(parts + 1) / 4.0e6;
		if (split > 0.85 * other)
			return false;
		plan.splits = static_cast<int>(parts);
		plan.steps_per_split = static_cast<int>(per_part);
		plan.bytes = static_cast<int64_t>(plane_bytes) * parts;
		return true;
	}
	template<typename TE>
	int launch_split(hipStream_t st, const avhipConvShape &s, const void *x, const void *w, const void *bias, const void *z, void *y, const void *padding_value,
			double alpha1, double alpha2, double beta, int activation, void *workspace, int64_t workspace_bytes)
	{
		SplitPlan plan;
		const int flags = vector_flags<TE>(s, x, w, y, z, sizeof(TE));
		if (!split_k_plan<TE>(s, plan) || !fast_path_ok<TE>(s, flags, padding_value) || (flags & 2) == 0 || workspace == nullptr
				|| workspace_bytes < plan.bytes || !aligned_to(workspace, 16))
			return AVHIP_NOT_SUPPORTED;
		const ConvGeom g = make_geom<TE>(s);
		const dim3 grid(ceil_div(g.pixels, BLOCK_M), ceil_div(s.K, BLOCK_N), static_cast<unsigned int>(plan.splits));
		hipLaunchKernelGGL((k_conv_igemm_split<TE>), grid, dim3(256), 0, st, static_cast<const TE*>(x), static_cast<const TE*>(w), g, plan.steps_per_split,
				static_cast<float*>(workspace));
		const FloatEpilogue<TE> epi { static_cast<const float*>(bias), static_cast<const TE*>(z), static_cast<TE*>(y), static_cast<float>(alpha1),
				static_cast<float>(alpha2), static_cast<float>(beta), activation, s.K, true };
		const int64_t plane = g.pixels * s.K;
		hipLaunchKernelGGL((k_split_reduce<TE>), dim3(ceil_div(plane / 4, 256)), dim3(256), 0, st, static_cast<const float*>(workspace), plan.splits, plane, epi);
		return 0;
	}
	bool shape_ok(const avhipConvShape *shape)
	{
		if (shape == nullptr)
			return false;
		const avhipConvShape &s = *shape;
		return s.N > 0 && s.H > 0 && s.W > 0 && s.C > 0 && s.K > 0 && s.R > 0 && s.S > 0 && s.Ho > 0 && s.Wo > 0 && s.stride_h > 0 && s.stride_w > 0 && s.dil_h > 0
				&& s.dil_w > 0 && (static_cast<int64_t>(s.K) + BLOCK_N - 1) / BLOCK_N <= 65535;
	}
}

extern "C" int avhip_conv2d_split_k_workspace(int x_dtype, const avhipConvShape *shape, int64_t *bytes)
{
	if (!shape_ok(shape) || bytes == nullptr)
		return AVHIP_BAD_PARAM;
	SplitPlan plan;
	bool yes = false;
	switch (x_dtype)
	{
		case DT_FLOAT32:
			yes = split_k_plan<float>(*shape, plan);
			break;
		case DT_FLOAT16:
			yes = split_k_plan<f16_t>(*shape, plan);
			break;
		case DT_BFLOAT16:
			yes = split_k_plan<bf16_t>(*shape, plan);
			break;
		default:
			break;
	}
	*bytes = yes ? plan.bytes : 0;
	return 0;
}

extern "C" int avhip_conv2d_implicit_gemm_split_k(void *stream, int x_dtype, const avhipConvShape *shape, const void *x, const void *w, const void *bias,
		const void *z, void *y, const void *padding_value, double alpha1, double alpha2, double beta, int activation, void *workspace, int64_t workspace_bytes)
{
	if (!shape_ok(shape) || x == nullptr || w == nullptr || y == nullptr)
		return AVHIP_BAD_PARAM;
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (x_dtype)
	{
		case DT_FLOAT32:
			return launch_split<float>(st, *shape, x, w, bias, z, y, padding_value, alpha1, alpha2, beta, activation, workspace, workspace_bytes);
		case DT_FLOAT16:
			return launch_split<f16_t>(st, *shape, x, w, bias, z, y, padding_value, alpha1, alpha2, beta, activation, workspace, workspace_bytes);
		case DT_BFLOAT16:
			return launch_split<bf16_t>(st, *shape, x, w, bias, z, y, padding_value, alpha1, alpha2, beta, activation, workspace, workspace_bytes);
		default:
			return AVHIP_NOT_SUPPORTED;
	}
}
