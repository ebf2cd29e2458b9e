/*
 * conv_pointwise.hip -- 1x1 convolutions (stride 1, no padding) as the persistent NT product
 * y[pixels, K] = x[pixels, C] * w[K, C]^T of persistent_gemm.hpp, with the convolution epilogue.
 *
 * Same arithmetic as the implicit-GEMM forward of the reference (src/conv2d_implicit_gemm.cu:152-301 with a one-tap
 * filter).  A 1x1 filter has a short k (C / 64 steps for 16-bit tensors) and x streams in from HBM once; the gather kernel's
 * one tile per workgroup leaves the matrix cores idle through every tile's first loads and drain.
 */
#include "conv_pointwise.hpp"
#include "persistent_gemm.hpp"
#include "resident_gemm.hpp"

namespace
{
	using namespace avhip;

	template<typename TE, typename Epi, int STEPS>
	__global__ __launch_bounds__(256, 2) void k_conv_pointwise(const TE *__restrict__ x, const TE *__restrict__ w, PersistentGeom g, Epi epi)
	{
		__shared__ __attribute__((aligned(16))) char lds[PERSISTENT_LDS_BYTES];
		persistent_nt_gemm<TE, Epi, STEPS>(lds, x, w, g, epi);
	}

	/* the same product with the filters resident in registers and only x streaming (resident_gemm.hpp) */
	template<typename TE, typename Epi, int STEPS>
	__global__ __launch_bounds__(256, RESIDENT_OCCUPANCY) void k_conv_pointwise_resident(const TE *__restrict__ x, const TE *__restrict__ w, ResidentGeom g, Epi epi)
	{
		__shared__ __attribute__((aligned(16))) char lds[RESIDENT_LDS_BYTES];
		resident_nt_gemm<TE, Epi, STEPS>(lds, x, w, g, epi);
	}
}

namespace avhip
{
	std::atomic<int>& short_k_engine()
	{
		static std::atomic<int> engine { 0 };
		return engine;
	}
}
extern "C" int avhip_set_short_k_engine(int engine)
{
	return avhip::short_k_engine().exchange(engine == 1 ? 1 : 0);
}

namespace avhip
{
	template<typename TE, typename Epi>
	bool conv_pointwise_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi)
	{
		if (s.R != 1 || s.S != 1 || s.stride_h != 1 || s.stride_w != 1 || s.pad_h != 0 || s.pad_w != 0 || s.Ho != s.H || s.Wo != s.W)
			return false;
		/* whole runs of Epi::wide filters leave with one vector store */
		if (!epi.vec || s.K % Epi::wide != 0 || !aligned_to(epi.y, 16) || (epi.z != nullptr && !aligned_to(epi.z, 16)))
			return false;
		if (static_cast<size_t>(s.K) * sizeof(typename Epi::template ColumnsT<1>) > static_cast<size_t>(PERSISTENT_TABLE_BYTES))
			return false;
		const int64_t pixels = static_cast<int64_t>(s.N) * s.H * s.W;
		const int64_t row_blocks = (pixels + BLOCK_M - 1) / BLOCK_M, col_blocks = (static_cast<int64_t>(s.K) + BLOCK_N - 1) / BLOCK_N;
		const int64_t tiles = row_blocks * col_blocks;
		if (pixels >= (1ll << 31) - BLOCK_M || tiles >= (1ll << 31) - 1024 || s.K >= (1 << 22))
			return false;
		const unsigned int x_row_bytes = static_cast<unsigned int>(s.C) * static_cast<unsigned int>(sizeof(TE));
		const int x_steps = static_cast<int>((x_row_bytes + STEP_BYTES - 1) / STEP_BYTES);
		if (short_k_engine().load(std::memory_order_relaxed) == 0 && x_steps <= RESIDENT_MAX_STEPS && x_row_bytes % 16 == 0
				&& static_cast<size_t>(s.K) * sizeof(typename Epi::template ColumnsT<1>) <= static_cast<size_t>(RESIDENT_TABLE_BYTES))
		{
			ResidentGeom r;
			r.rows = static_cast<int>(pixels);
			r.cols = s.K;
			r.row_bytes = x_row_bytes;
			r.a_pitch = r.b_pitch = x_row_bytes;
			r.a_batch = r.b_batch = 0;
			r.a_bytes = static_cast<unsigned int>(pixels) * x_row_bytes; /* the caller vouches for tensors below 2 GiB */
			r.b_bytes = static_cast<unsigned int>(s.K) * x_row_bytes;
			r.c_batch = 0;
			r.c_pitch = s.K;
			r.table_columns = s.K;
			const dim3 grid(resident_plan(r, 1));
			const TE *xp = static_cast<const TE*>(x), *wp = static_cast<const TE*>(w);
			if (x_steps == 1)
				hipLaunchKernelGGL((k_conv_pointwise_resident<TE, Epi, 1>), grid, dim3(256), 0, stream, xp, wp, r, epi);
			else if (x_steps == 2)
				hipLaunchKernelGGL((k_conv_pointwise_resident<TE, Epi, 2>), grid, dim3(256), 0, stream, xp, wp, r, epi);
			else
				hipLaunchKernelGGL((k_conv_pointwise_resident<TE, Epi, 4>), grid, dim3(256), 0, stream, xp, wp, r, epi);
			return true;
		}
		PersistentGeom g;
		g.rows = static_cast<int>(pixels);
		g.cols = s.K;
		g.row_bytes = static_cast<unsigned int>(s.C) * static_cast<unsigned int>(sizeof(TE));
		const int steps = static_cast<int>((g.row_bytes + STEP_BYTES - 1) / STEP_BYTES);
		/* a register set of x per step: longer rows stay with the gather kernel, whose k loop is long enough (int8 gets two
		 * sets: its epilogue constants take the registers the other two would need) */
		constexpr int MAX_STEPS = sizeof(TE) == 1 ? 2 : PERSISTENT_MAX_STEPS;
		if (steps > MAX_STEPS)
			return false;
		g.a_pitch = g.b_pitch = g.row_bytes;
		g.a_batch = g.b_batch = 0;
		g.a_bytes = static_cast<unsigned int>(pixels) * g.row_bytes; /* the caller vouches for tensors below 2 GiB */
		g.b_bytes = static_cast<unsigned int>(s.K) * g.row_bytes;
		g.c_batch = 0;
		g.c_pitch = s.K;
		g.row_blocks = static_cast<int>(row_blocks);
		g.col_blocks = static_cast<int>(col_blocks);
		g.tiles = static_cast<int>(tiles);
		g.table_columns = s.K;
		const dim3 grid(persistent_workgroups(tiles));
		if (steps <= 2)
			hipLaunchKernelGGL((k_conv_pointwise<TE, Epi, 2>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		else if constexpr (MAX_STEPS >= 4)
			hipLaunchKernelGGL((k_conv_pointwise<TE, Epi, 4>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		return true;
	}

#define AVHIP_INSTANTIATE(TE, EPI) template bool conv_pointwise_launch<TE, EPI>(hipStream_t, const avhipConvShape&, const void*, const void*, const EPI&);
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
