/*
 * conv_small.hip -- implicit-GEMM convolution for problems too small to fill the chip with 128 x 128 workgroup tiles.
 *
 * A batch of 8 images of 15 x 15 pixels with 64 filters is 15 tiles of 128 x 128: 15 of 256 compute units busy, each for the
 * whole k range.  This kernel cuts the same GEMM (rows = output pixels, columns = filters, k = (tap, channel)) into
 * 32 x 32 tiles, one per WAVEFRONT (workgroup = 64 work-items), several hundred of them for such a problem, and drops
 * everything a small problem does not need: no LDS staging, no barriers in the k loop.  Each lane fetches its own MFMA
 * operands straight from global memory in the operand layout (lane l: row l % 32 of the tile, 16-byte k-chunk l / 32 of a
 * 32-byte slab) with out-of-range buffer loads for padding and tails; the re-use of x and w between wavefronts is left to
 * L2, which holds a small problem entirely.  Loads run one group of four slabs ahead of the MFMAs.  The accumulator tile
 * leaves through 4 KB of LDS so that a lane stores four consecutive filters of a pixel, with the shared epilogue.
 */
#include <atomic>

#include "conv_small.hpp"
#include "mfma_core.hpp"

namespace
{
	using namespace avhip;

	constexpr int SMALL_TILE = 32;
	constexpr int GROUP = 4; /* 32-byte k-slabs fetched together */
	constexpr int SMALL_PITCH = SMALL_TILE + 4; /* words per LDS row of the drain buffer */

	struct SmallGeom
	{
		int H, W, C, K, R, S, Ho, Wo, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, flip;
		int slabs_per_tap; /* 32-byte slabs covering the channels of one tap */
		int pixels, images;
	};

	/* KW wavefronts share one tile: each takes a contiguous KW-th of the k range and the partial tiles are summed through LDS.
	 * KW = 4 when even the 32 x 32 tiling leaves most SIMDs without a wavefront. */
	template<typename TE, typename Epi, int KW>
	__global__ __launch_bounds__(64 * KW) void k_conv_small(const TE *__restrict__ x, const TE *__restrict__ w, SmallGeom g, Epi epi)
	{
		__shared__ __attribute__((aligned(16))) typename Epi::scalar_t sm[KW * SMALL_TILE * SMALL_PITCH];
		constexpr unsigned int SZ = sizeof(TE);
		const int lane = threadIdx.x & 63;
		const int wave = threadIdx.x >> 6;
		const int r = lane & 31;
		const unsigned int half = (lane >> 5) * 16;
		/* neighbouring pixel tiles read overlapping windows: a contiguous run of them goes to one XCD and its L2 */
		const int p0 = static_cast<int>(xcd_block(blockIdx.x, gridDim.x)) * SMALL_TILE, k0 = blockIdx.y * SMALL_TILE;
		const int kcol = k0 + (threadIdx.x & 7) * 4;
		typename Epi::Columns columns;
		epi.load_columns(kcol, columns);

		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, static_cast<unsigned int>(g.images) * g.H * g.W * g.C * SZ);
		const __amdgpu_buffer_rsrc_t rw = make_buffer(w, static_cast<unsigned int>(g.K) * g.R * g.S * g.C * SZ);
		const unsigned int c_bytes = g.C * SZ;

		/* this lane's row of A: one output pixel */
		const int p = p0 + r;
		const bool row_ok = p < g.pixels;
		const int pp = row_ok ? p : 0;
		const int line = pp / g.Wo, ow = pp - line * g.Wo;
		const int n = line / g.Ho, oh = line - n * g.Ho;
		const int ih0 = oh * g.stride_h + g.pad_h, iw0 = ow * g.stride_w + g.pad_w;
		const unsigned int a_origin = static_cast<unsigned int>((n * g.H + ih0) * g.W + iw0) * c_bytes + half;
		unsigned int inside = 0;
		if (row_ok)
		{
			unsigned int cols = 0;
			for (int j = 0; j < g.S; j++)
			{
				const int iw = iw0 + (g.flip ? g.S - 1 - j : j) * g.dil_w;
				if (iw >= 0 && iw < g.W)
					cols |= 1u << j;
			}
			for (int i = 0; i < g.R; i++)
			{
				const int ih = ih0 + (g.flip ? g.R - 1 - i : i) * g.dil_h;
				if (ih >= 0 && ih < g.H)
					inside |= cols << (i * g.S);
			}
		}
		/* this lane's row of B: one filter */
		const int kf = k0 + r;
		const unsigned int b_origin = kf < g.K ? static_cast<unsigned int>(kf) * g.R * g.S * c_bytes + half : OUT_OF_RANGE;

		typename Mma<TE>::acc_t acc;
#pragma unroll
		for (int v = 0; v < 16; v++)
			acc[v] = 0;

		/* k walks (tap, slab); everything about the position is wavefront-uniform */
		const int taps = g.R * g.S;
		const int groups_all = (taps * g.slabs_per_tap + GROUP - 1) / GROUP;
		const int groups = (groups_all + KW - 1) / KW; /* groups of this wavefront: [wave * groups, (wave + 1) * groups) */
		const int first_slab = wave * groups * GROUP;
		int f_tap = first_slab / g.slabs_per_tap, f_slab = first_slab - f_tap * g.slabs_per_tap;
		int f_i = f_tap / g.S, f_j = f_tap - f_i * g.S;
		int left = groups * GROUP; /* slabs this wavefront may still fetch */
		auto fetch = [&](uint4 (&a)[GROUP], uint4 (&b)[GROUP]) __attribute__((always_inline))
		{
#pragma unroll
			for (int q = 0; q < GROUP; q++)
			{
				const int i = g.flip ? g.R - 1 - f_i : f_i, j = g.flip ? g.S - 1 - f_j : f_j;
				const unsigned int cb = static_cast<unsigned int>(f_slab) * 32u;
				const bool live = (left > 0) & (f_tap < taps) & (cb + half < c_bytes);
				left--;
				const unsigned int a_tap = static_cast<unsigned int>((i * g.dil_h) * g.W + j * g.dil_w) * c_bytes + cb;
				const unsigned int b_tap = static_cast<unsigned int>(f_tap) * c_bytes + cb;
				a[q] = buffer_fetch(rx, (live && ((inside >> (f_tap & 31)) & 1u)) ? a_origin + a_tap : OUT_OF_RANGE);
				b[q] = buffer_fetch(rw, (live && b_origin != OUT_OF_RANGE) ? b_origin + b_tap : OUT_OF_RANGE);
				if (++f_slab == g.slabs_per_tap)
				{
					f_slab = 0;
					f_tap++;
					if (++f_j == g.S)
					{
						f_j = 0;
						f_i++;
					}
				}
			}
		};
		auto multiply = [&](const uint4 (&a)[GROUP], const uint4 (&b)[GROUP]) __attribute__((always_inline))
		{
#pragma unroll
			for (int q = 0; q < GROUP; q++)
			{
				Chunk ca, cb;
				ca.u = a[q];
				cb.u = b[q];
				Mma<TE>::run(ca, cb, acc);
			}
		};
		uint4 a0[GROUP], b0[GROUP], a1[GROUP], b1[GROUP];
		fetch(a0, b0);
		for (int s = 0; s < groups; s += 2)
		{
			fetch(a1, b1); /* zeros past the last slab */
			multiply(a0, b0);
			fetch(a0, b0);
			multiply(a1, b1);
		}

		/* lane holds column r, rows 8 i + 4 (lane / 32) + j of its wavefront's partial tile; after the transpose through LDS a
		 * work-item owns 4 consecutive columns of a row and adds up the KW partial tiles */
		typename Epi::scalar_t *mine = sm + wave * (SMALL_TILE * SMALL_PITCH);
#pragma unroll
		for (int i = 0; i < 4; i++)
#pragma unroll
			for (int j = 0; j < 4; j++)
				mine[(8 * i + 4 * (lane >> 5) + j) * SMALL_PITCH + r] = acc[4 * i + j];
		__syncthreads();
#pragma unroll
		for (int it = 0; it < 4 / KW; it++)
		{
			const int row = (static_cast<int>(threadIdx.x) >> 3) + 8 * KW * it;
			typedef Pack<typename Epi::scalar_t, 4> P4;
			P4 v = *reinterpret_cast<const P4*>(sm + row * SMALL_PITCH + (threadIdx.x & 7) * 4);
#pragma unroll
			for (int part = 1; part < KW; part++)
			{
				const P4 o = *reinterpret_cast<const P4*>(sm + part * (SMALL_TILE * SMALL_PITCH) + row * SMALL_PITCH + (threadIdx.x & 7) * 4);
#pragma unroll
				for (int q = 0; q < 4; q++)
					v.v[q] += o.v[q];
			}
			if (p0 + row < g.pixels && kcol < g.K)
				epi.template store<ACT_SIMPLE, true>(p0 + row, kcol, v.v, columns);
		}
	}
}

namespace
{
	/* below this many big workgroups most of the 256 compute units would idle */
	std::atomic<int>& small_problem_threshold()
	{
		static std::atomic<int> value(192);
		return value;
	}
}

extern "C" int avhip_set_small_problem_threshold(int workgroups)
{
	return small_problem_threshold().exchange(workgroups < 0 ? -1 : workgroups);
}

namespace avhip
{
	/* Small in tiles is not enough: the problem must be short in k as well.  A wavefront fetches its own operands, one 32-byte
	 * slab of both per MFMA with no re-use inside a workgroup: measured about 0.12 us per slab, plus 0.19 us per slab and
	 * wavefront per SIMD as the tiles crowd L2 (a 3x3 layer of 256 channels on 32 images of 14 x 14 took 59 us here and 19 us in
	 * the image-tile kernel with half the compute units idle).  The workgroup-tile kernels take about 0.7 us per 128-byte
	 * k-step and 4 us around the loop, per round of 512 workgroups. */
	SmallProblemEstimate conv_small_estimate(const avhipConvShape &s, int element_bytes, int64_t big_tile_workgroups)
	{
		const int64_t pixels = static_cast<int64_t>(s.N) * s.Ho * s.Wo;
		const int64_t tiles = ((pixels + SMALL_TILE - 1) / SMALL_TILE) * ((static_cast<int64_t>(s.K) + SMALL_TILE - 1) / SMALL_TILE);
		const int slabs_per_tap = (s.C * element_bytes + 31) / 32;
		SmallProblemEstimate e;
		/* fewer tiles than half the 1024 SIMDs of the chip, and enough k to share: four wavefronts per tile */
		e.split_k = tiles < 512 && static_cast<int64_t>(s.R) * s.S * slabs_per_tap >= 4 * GROUP;
		const double wavefronts = static_cast<double>(tiles) * (e.split_k ? 4 : 1);
		const double slabs = static_cast<double>(s.R) * s.S * slabs_per_tap / (e.split_k ? 4 : 1);
		e.small_us = 2.5 + slabs * (0.12 + 0.19 * wavefronts / 1024.0);
		const double k_steps = static_cast<double>(s.R) * s.S * ((s.C * element_bytes + 127) / 128);
		e.workgroup_tiles_us = static_cast<double>((big_tile_workgroups + 511) / 512) * (0.7 * k_steps + 4.0);
		return e;
	}
	bool conv_small_preferred(const avhipConvShape &s, int element_bytes, int64_t big_tile_workgroups)
	{
		const int64_t busy = small_problem_threshold().load(std::memory_order_relaxed);
		if (busy < 0) /* asked for by name (tests): whatever the kernel can run */
			return true;
		if (big_tile_workgroups >= busy)
			return false;
		const SmallProblemEstimate e = conv_small_estimate(s, element_bytes, big_tile_workgroups);
		return e.small_us <= e.workgroup_tiles_us;
	}

	template<typename TE, typename Epi>
	bool conv_small_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi, int64_t big_tile_workgroups)
	{
		const int64_t pixels = static_cast<int64_t>(s.N) * s.Ho * s.Wo;
		if (!conv_small_preferred(s, static_cast<int>(sizeof(TE)), big_tile_workgroups) || !epi.vec || s.R * s.S > 32)
			return false;
		const int64_t tiles = (pixels + SMALL_TILE - 1) / SMALL_TILE, filter_tiles = (static_cast<int64_t>(s.K) + SMALL_TILE - 1) / SMALL_TILE;
		if (tiles > 0x7FFFFFFFll || filter_tiles > 65535 || pixels >= (1ll << 31) - SMALL_TILE)
			return false;
		const int slabs_per_tap = (s.C * static_cast<int>(sizeof(TE)) + 31) / 32;
		const bool split_k = conv_small_estimate(s, static_cast<int>(sizeof(TE)), big_tile_workgroups).split_k;
		SmallGeom g;
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
		g.flip = s.mode != 0 ? 1 : 0;
		g.slabs_per_tap = slabs_per_tap;
		g.pixels = static_cast<int>(pixels);
		g.images = s.N;
		const dim3 grid(static_cast<unsigned int>(tiles), static_cast<unsigned int>(filter_tiles));
		/* fewer tiles than half the 1024 SIMDs of the chip, and enough k to share: four wavefronts per tile */
		if (split_k)
			hipLaunchKernelGGL((k_conv_small<TE, Epi, 4>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		else
			hipLaunchKernelGGL((k_conv_small<TE, Epi, 1>), grid, dim3(64), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		return true;
	}

#define AVHIP_INSTANTIATE(TE, EPI) template bool conv_small_launch<TE, EPI>(hipStream_t, const avhipConvShape&, const void*, const void*, const EPI&, int64_t);
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
