/*
 * conv_stem.hip -- implicit-GEMM convolution for the first layer of a tower: very few input channels, a small filter.
 *
 * Same arithmetic as the implicit-GEMM forward of the reference (src/conv2d_implicit_gemm.cu:152-301).  With 4 input planes
 * and a 3 x 3 filter the whole k extent is 36 elements: there is no k loop to pipeline, the layer is a pure stream of output
 * (N*Ho*Wo*K elements written for almost nothing read), and what a general kernel spends on it is latency: address set-up
 * for a gather it runs once, a trip through LDS for operands that are used once, workgroup barriers around one step.
 * Here a wavefront works alone: the MFMA operands come straight from memory into registers in the layout the matrix
 * cores take (a lane's 16-byte chunk of the A operand is two neighbouring taps of one pixel, two 8-byte loads; pixels outside
 * the image ask for an out-of-range offset and get zeros), the filters are read once per wavefront, twelve MFMAs produce
 * 64 pixels x 64 filters, and the accumulators leave through the wavefront's own LDS region as whole 16-byte runs of
 * filters per pixel with bias / residual / ReLU applied.  No workgroup-level hand-over except the one barrier the drain
 * starts with.
 */
#include "conv_stem.hpp"
#include "mfma_core.hpp"
#include <type_traits>

namespace
{
	using namespace avhip;

	constexpr int STEM_MAX_TAPS = 12; /* three MFMA slabs of four taps */
	constexpr int STEM_SLABS = STEM_MAX_TAPS / 4;
	constexpr unsigned int STEM_NO_TAP = 0x7FFF0000u; /* a row offset no image reaches */

	struct StemGeom
	{
		int H, W, K, Ho, Wo, pad_h, pad_w, stride_h, stride_w;
		int pixels; /* N * Ho * Wo */
		unsigned int x_bytes, w_bytes, row_bytes; /* row_bytes: one filter = taps * 8 */
		unsigned int tap_yx[STEM_MAX_TAPS]; /* (row offset << 16) | column offset of the input pixel a filter tap multiplies */
	};

	__device__ inline uint2 buffer_fetch8(__amdgpu_buffer_rsrc_t rsrc, unsigned int byte_offset)
	{
		typedef __attribute__((__vector_size__(2 * sizeof(unsigned int)))) unsigned int u32x2_t;
		const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, static_cast<int>(byte_offset), 0, 0);
		return make_uint2(v[0], v[1]);
	}

	template<typename TE, typename Epi>
	__global__ __launch_bounds__(256, 2) void k_conv_stem(const TE *__restrict__ x, const TE *__restrict__ w, StemGeom g, Epi epi)
	{
		epi.pin();
		constexpr int W = Epi::wide;
		typedef PrivateDrainRows<2, W> Rows;
		__shared__ __attribute__((aligned(16))) char lds[4 * Rows::bytes];
		const int lane = threadIdx.x & 63;
		const int wave = threadIdx.x >> 6;
		const int half = lane >> 5; /* which 16 bytes of a 32-byte slab this lane supplies */
		const int p0 = static_cast<int>(blockIdx.x) * 256;
		const int k0 = static_cast<int>(blockIdx.y) * 64;
		const int kcol = k0 + drain_column<1, W>();
		typename Epi::template ColumnsT<W> columns;
		epi.load_columns(kcol, columns);

		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, g.x_bytes);
		const __amdgpu_buffer_rsrc_t rw = make_buffer(w, g.w_bytes);

		/* filters: lane supplies filter (lane % 32) of a 32-filter tile; a filter row is `row_bytes` long and the chunk that
		 * straddles its end is cut (what follows belongs to the next filter) */
		Chunk b[2][STEM_SLABS];
#pragma unroll
		for (int tn = 0; tn < 2; tn++)
		{
			const int f = k0 + tn * 32 + (lane & 31);
#pragma unroll
			for (int s = 0; s < STEM_SLABS; s++)
			{
				const unsigned int in_row = 32u * s + 16u * half;
				const bool exists = f < g.K && in_row < g.row_bytes;
				b[tn][s].u = buffer_fetch(rw, exists ? static_cast<unsigned int>(f) * g.row_bytes + in_row : OUT_OF_RANGE);
				if (in_row + 8 >= g.row_bytes)
					b[tn][s].u.z = b[tn][s].u.w = 0;
			}
		}
		/* pixels: lane supplies output pixel (lane % 32) of a 32-pixel tile and the taps 4 s + 2 half, 4 s + 2 half + 1 */
		Chunk a[2][STEM_SLABS];
		const int plane = g.Ho * g.Wo;
#pragma unroll
		for (int tm = 0; tm < 2; tm++)
		{
			const int p = p0 + wave * 64 + tm * 32 + (lane & 31);
			const int n = p / plane, rest = p - n * plane;
			const int oh = rest / g.Wo, ow = rest - oh * g.Wo;
			const int h0 = oh * g.stride_h + g.pad_h, w0 = ow * g.stride_w + g.pad_w;
#pragma unroll
			for (int s = 0; s < STEM_SLABS; s++)
			{
				uint2 piece[2];
#pragma unroll
				for (int e = 0; e < 2; e++)
				{
					const unsigned int yx = half ? g.tap_yx[4 * s + 2 + e] : g.tap_yx[4 * s + e];
					const int ih = h0 + static_cast<int>(yx >> 16), iw = w0 + static_cast<int>(yx & 0xFFFFu);
					const bool inside = (p < g.pixels) & (ih >= 0) & (ih < g.H) & (iw >= 0) & (iw < g.W);
					piece[e] = buffer_fetch8(rx, inside ? static_cast<unsigned int>((n * g.H + ih) * g.W + iw) * 8u : OUT_OF_RANGE);
				}
				a[tm][s].u = make_uint4(piece[0].x, piece[0].y, piece[1].x, piece[1].y);
			}
		}

		typename Mma<TE>::acc_t acc[2][2];
#pragma unroll
		for (int i = 0; i < 2; i++)
#pragma unroll
			for (int j = 0; j < 2; j++)
#pragma unroll
				for (int v = 0; v < 16; v++)
					acc[i][j][v] = 0;
#pragma unroll
		for (int s = 0; s < STEM_SLABS; s++)
#pragma unroll
			for (int tm = 0; tm < 2; tm++)
#pragma unroll
				for (int tn = 0; tn < 2; tn++)
					Mma<TE>::run(a[tm][s], b[tn][s], acc[tm][tn]);

		if constexpr (std::is_same<Epi, FloatEpilogue<TE>>::value && sizeof(TE) == 2)
		{
			/* the usual first layer (16-bit tensors, no residual, beta = 0): no branch in the epilogue, rows past the end go to an
			 * out-of-range offset of a buffer over the 256 pixels of this workgroup, runs are written through as they go */
			if (epi.z == nullptr && epi.beta == 0.0f && g.K < (1 << 22))
			{
				constexpr unsigned int SZ = sizeof(TE);
				const __amdgpu_buffer_rsrc_t ry = make_buffer(epi.y + static_cast<int64_t>(p0) * g.K, 0x7FFFFFF0u);
				auto drain = [&](auto relu) __attribute__((always_inline))
				{
					drain_tile_private<TE, 2, W>(lds, acc, [&](int row, const float (&v)[W], int) __attribute__((always_inline))
					{
						const unsigned int offset = (p0 + row < g.pixels && kcol < g.K) ? static_cast<unsigned int>(row * g.K + kcol) * SZ : OUT_OF_RANGE;
						typename Epi::template Residual<W> none;
						epi.template store_fast<decltype(relu)::value, false, W>(v, columns, none, [&](auto words) __attribute__((always_inline))
						{
							buffer_put<STORE_STREAM_THROUGH>(ry, offset, words);
						});
					});
				};
				if (epi.activation == ACT_RELU)
					drain(std::true_type());
				else
					drain(std::false_type());
				return;
			}
		}
		drain_tile_private<TE, 2, W>(lds, acc, [&](int row, const typename Epi::scalar_t (&v)[W], int) __attribute__((always_inline))
		{
			const int p = p0 + row;
			if (p < g.pixels && kcol < g.K)
				epi.template store_at<ACT_SIMPLE, true, W>(static_cast<int64_t>(p) * g.K + kcol, kcol, v, columns, nullptr);
		});
	}
}

namespace avhip
{
	template<typename TE, typename Epi>
	bool conv_stem_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi)
	{
		/* the 16-byte operand chunk must be two pixels: 16-bit and 8-bit types */
		if constexpr (sizeof(TE) > 2)
			return false;
		else
		{
		const int taps = s.R * s.S;
		if (s.C * static_cast<int>(sizeof(TE)) != 8 || taps > STEM_MAX_TAPS)
			return false;
		if (s.H >= 16384 || s.W >= 16384 || (s.R - 1) * s.dil_h >= 16384 || (s.S - 1) * s.dil_w >= 16384)
			return false;
		/* whole runs of Epi::wide filters leave with one vector store */
		if (!epi.vec || s.K % Epi::wide != 0 || !aligned_to(epi.y, 16) || (epi.z != nullptr && !aligned_to(epi.z, 16)) || !aligned_to(x, 8) || !aligned_to(w, 4))
			return false;
		const int64_t pixels = static_cast<int64_t>(s.N) * s.Ho * s.Wo;
		const int64_t x_bytes = static_cast<int64_t>(s.N) * s.H * s.W * 8, w_bytes = static_cast<int64_t>(s.K) * taps * 8;
		const int64_t filter_blocks = (static_cast<int64_t>(s.K) + 63) / 64;
		if (pixels >= (1ll << 31) - 256 || x_bytes >= (1ll << 31) || w_bytes >= (1ll << 31) || filter_blocks > 65535)
			return false;
		StemGeom g;
		g.H = s.H;
		g.W = s.W;
		g.K = s.K;
		g.Ho = s.Ho;
		g.Wo = s.Wo;
		g.pad_h = s.pad_h;
		g.pad_w = s.pad_w;
		g.stride_h = s.stride_h;
		g.stride_w = s.stride_w;
		g.pixels = static_cast<int>(pixels);
		g.x_bytes = static_cast<unsigned int>(x_bytes);
		g.w_bytes = static_cast<unsigned int>(w_bytes);
		g.row_bytes = static_cast<unsigned int>(taps) * 8u;
		for (int t = 0; t < STEM_MAX_TAPS; t++)
		{
			g.tap_yx[t] = STEM_NO_TAP;
			if (t < taps)
			{
				/* filter tap (i, j) multiplies the input at (i, j), or at (R - 1 - i, S - 1 - j) when the kernel is flipped */
				const int i = t / s.S, j = t % s.S;
				const int dy = (s.mode != 0 ? s.R - 1 - i : i) * s.dil_h, dx = (s.mode != 0 ? s.S - 1 - j : j) * s.dil_w;
				g.tap_yx[t] = (static_cast<unsigned int>(dy) << 16) | static_cast<unsigned int>(dx);
			}
		}
		const dim3 grid(static_cast<unsigned int>((pixels + 255) / 256), static_cast<unsigned int>(filter_blocks));
		hipLaunchKernelGGL((k_conv_stem<TE, Epi>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		return true;
		}
	}

#define AVHIP_INSTANTIATE(TE, EPI) template bool conv_stem_launch<TE, EPI>(hipStream_t, const avhipConvShape&, const void*, const void*, const EPI&);
	AVHIP_INSTANTIATE(float, FloatEpilogue<float>)
	AVHIP_INSTANTIATE(f16_t, FloatEpilogue<f16_t>)
	AVHIP_INSTANTIATE(bf16_t, FloatEpilogue<bf16_t>)
	AVHIP_INSTANTIATE(int8_t, Int8Epilogue<I8_EXACT>)
	AVHIP_INSTANTIATE(int8_t, Int8Epilogue<I8_REQUANT>)
	AVHIP_INSTANTIATE(int8_t, Int8Epilogue<I8_FLOAT_I32>)
	AVHIP_INSTANTIATE(int8_t, Int8Epilogue<I8_FLOAT_I8>)
	AVHIP_INSTANTIATE(int8_t, Int8Epilogue<I8_FLOAT_F32>)
#undef AVHIP_INSTANTIATE
}
