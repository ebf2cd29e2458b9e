/*
 * conv_pointwise.hip -- 1x1 convolutions (stride 1, no padding) as a persistent NT GEMM  y[pixels, K] = x[pixels, C] * w[K, C]^T.
 *
 * Same arithmetic as the implicit-GEMM forward of the reference (src/conv2d_implicit_gemm.cu:152-301 with a one-tap
 * filter); same 128 x 128 workgroup tile, MFMA shapes, LDS layout and epilogue as the gather kernel.  What differs is the
 * schedule.  A 1x1 filter has a short k (C / 64 steps for 16-bit tensors) and x streams in from HBM: a workgroup that
 * computes one tile spends most of its life waiting for its first operands and draining its accumulators.  Here a workgroup
 * stays on its compute unit and walks a sequence of tiles as ONE software pipeline:
 *   - x: every k-step of a tile has its own register set, and a set is refilled with the same step of the NEXT tile right
 *     after it went to LDS, so the x of a tile is requested before the previous tile is drained;
 *   - w: comes from L2 (it is small and shared by everybody) two k-steps ahead, across tile boundaries (a register set per
 *     step for w as well spills and was measured slower);
 *   - the accumulators of a finished tile leave through the LDS buffer that tile no longer needs while the other buffer
 *     already holds the first step of the next tile;
 *   - per-filter constants (bias, scale) sit in LDS for all filters: nothing of a tile waits on the memory counter but its
 *     own operands.
 * Tiles are numbered with the filter block fastest and each XCD takes a contiguous run of them, so the workgroups that
 * share a block of pixels run at the same time behind the same L2 and x comes from HBM once.
 */
#include "conv_pointwise.hpp"
#include "mfma_core.hpp"

namespace
{
	using namespace avhip;

	constexpr int TABLE_BYTES = 8192; /* LDS left for the per-filter constants with two workgroups per compute unit */

	struct PointGeom
	{
		int pixels, K;
		unsigned int row_bytes; /* C * sizeof(TE) */
		int filter_blocks; /* ceil(K / 128) */
		int tiles; /* pixel blocks * filter blocks */
	};

	/* STEPS: k-steps per tile, even (an odd count is rounded up and the extra step reads zeros). */
	template<typename TE, typename Epi, int STEPS>
	__global__ __launch_bounds__(256, 2) void k_conv_pointwise(const TE *__restrict__ x, const TE *__restrict__ w, PointGeom g, Epi epi)
	{
		static_assert(STEPS % 2 == 0, "register sets and LDS buffers alternate with the step parity");
		__shared__ __attribute__((aligned(16))) char lds[LDS_BYTES + TABLE_BYTES];
		constexpr int W = Epi::wide;
		static_assert(DrainShape<2, W>::bytes <= 2 * LDS_TILE, "the accumulators leave through one operand buffer");
		typedef typename Epi::template ColumnsT<1> Record;
		Record *table = reinterpret_cast<Record*>(lds + LDS_BYTES);
		epi.pin();
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wm = wave >> 1, wn = wave & 1;
		const int fpart = tid & (STEP_CHUNKS - 1);
		const int frow = tid / STEP_CHUNKS;
		const int st_off = frow * LDS_ROW + fpart * 16;
		const int rd_a = (wm * 64 + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;
		const int rd_b = (wn * 64 + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;
		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, static_cast<unsigned int>(g.pixels) * g.row_bytes);
		const __amdgpu_buffer_rsrc_t rw = make_buffer(w, static_cast<unsigned int>(g.K) * g.row_bytes);

		/* tile sequence of this workgroup: round j takes tile j * gridDim.x + (its number within the round, XCD-contiguous) */
		const int first = xcd_block(blockIdx.x, gridDim.x);
		const int stride = gridDim.x;
		auto pixel_block = [&](int tile) { return static_cast<int>(static_cast<unsigned int>(tile) / static_cast<unsigned int>(g.filter_blocks)); };

		/* the two fetch cursors: x one tile ahead of the MFMAs, w two steps ahead */
		int a_tile = first, a_step = 0, b_tile = first, b_step = 0;
		unsigned int a_base[FETCH_PASSES], b_base[FETCH_PASSES];
		auto aim_a = [&]()
		{
			const bool live = a_tile < g.tiles;
			const int pb = live ? pixel_block(a_tile) : 0;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int p = pb * BLOCK_M + frow + FETCH_ROWS * q;
				a_base[q] = (live && p < g.pixels) ? static_cast<unsigned int>(p) * g.row_bytes + fpart * 16 : OUT_OF_RANGE;
			}
		};
		auto aim_b = [&]()
		{
			const bool live = b_tile < g.tiles;
			const int kb = live ? b_tile - pixel_block(b_tile) * g.filter_blocks : 0;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int k = kb * BLOCK_N + frow + FETCH_ROWS * q;
				b_base[q] = (live && k < g.K) ? static_cast<unsigned int>(k) * g.row_bytes + fpart * 16 : OUT_OF_RANGE;
			}
		};
		auto fetch_a = [&](uint4 (&a)[FETCH_PASSES]) __attribute__((always_inline))
		{
			const unsigned int k_byte = static_cast<unsigned int>(a_step) * STEP_BYTES;
			const bool in_row = k_byte + fpart * 16 < g.row_bytes;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
				a[q] = buffer_fetch(rx, (in_row && a_base[q] < OUT_OF_RANGE) ? a_base[q] + k_byte : OUT_OF_RANGE);
			if (++a_step == STEPS)
			{
				a_step = 0;
				a_tile += stride;
				aim_a();
			}
		};
		auto fetch_b = [&](uint4 (&b)[FETCH_PASSES]) __attribute__((always_inline))
		{
			const unsigned int k_byte = static_cast<unsigned int>(b_step) * STEP_BYTES;
			const bool in_row = k_byte + fpart * 16 < g.row_bytes;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
				b[q] = buffer_fetch(rw, (in_row && b_base[q] < OUT_OF_RANGE) ? b_base[q] + k_byte : OUT_OF_RANGE);
			if (++b_step == STEPS)
			{
				b_step = 0;
				b_tile += stride;
				aim_b();
			}
		};
		auto stash = [&](int buffer, const uint4 (&a)[FETCH_PASSES], const uint4 (&b)[FETCH_PASSES]) __attribute__((always_inline))
		{
			char *sa = lds + buffer * 2 * LDS_TILE;
			char *sb = sa + LDS_TILE;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				*reinterpret_cast<uint4*>(sa + st_off + q * FETCH_ROWS * LDS_ROW) = a[q];
				*reinterpret_cast<uint4*>(sb + st_off + q * FETCH_ROWS * LDS_ROW) = b[q];
			}
		};

		typename Mma<TE>::acc_t acc[2][2];
		auto multiply = [&](int buffer) __attribute__((always_inline))
		{
			const char *sa = lds + buffer * 2 * LDS_TILE;
			const char *sb = sa + LDS_TILE;
			constexpr int SLABS = STEP_BYTES / 32;
			Chunk a[2][2], b[2][2]; /* LDS reads run one 32-byte slab ahead of the MFMAs */
			auto read = [&](int slab, Chunk (&ra_)[2], Chunk (&rb_)[2]) __attribute__((always_inline))
			{
#pragma unroll
				for (int i = 0; i < 2; i++)
				{
					ra_[i].u = *reinterpret_cast<const uint4*>(sa + rd_a + i * 32 * LDS_ROW + slab * 32);
					rb_[i].u = *reinterpret_cast<const uint4*>(sb + rd_b + i * 32 * LDS_ROW + slab * 32);
				}
			};
			read(0, a[0], b[0]);
#pragma unroll
			for (int slab = 0; slab < SLABS; slab++)
			{
				if (slab + 1 < SLABS)
					read(slab + 1, a[(slab + 1) & 1], b[(slab + 1) & 1]);
				if (sizeof(TE) < 4)
					__builtin_amdgcn_s_setprio(1);
#pragma unroll
				for (int i = 0; i < 2; i++)
#pragma unroll
					for (int j = 0; j < 2; j++)
						Mma<TE>::run(a[slab & 1][i], b[slab & 1][j], acc[i][j]);
				if (sizeof(TE) < 4)
					__builtin_amdgcn_s_setprio(0);
			}
		};

		/* prologue: all of the first tile's x, two steps of w, step 0 into LDS, and set 0 of x goes on to the second tile */
		uint4 ra[STEPS][FETCH_PASSES], rb[2][FETCH_PASSES];
		aim_a();
		aim_b();
#pragma unroll
		for (int s = 0; s < STEPS; s++)
			fetch_a(ra[s]);
		fetch_b(rb[0]);
		fetch_b(rb[1]);
		for (int k = tid; k < g.K; k += 256)
			epi.load_columns(k, table[k]);
		stash(0, ra[0], rb[0]);
		fetch_a(ra[0]);

		const int col = drain_column<2, W>();
		for (int tile = first; tile < g.tiles; tile += stride)
		{
			const int pb = pixel_block(tile);
			const int k = (tile - pb * g.filter_blocks) * BLOCK_N + col;
#pragma unroll
			for (int i = 0; i < 2; i++)
#pragma unroll
				for (int j = 0; j < 2; j++)
#pragma unroll
					for (int v = 0; v < 16; v++)
						acc[i][j][v] = 0;
			/* step s is multiplied from LDS buffer s % 2; meanwhile step s + 2 of w is requested into the set step s just
			 * left, step s + 1 goes to the other buffer, and the x set it came from is refilled for the next tile */
#pragma unroll
			for (int s = 0; s < STEPS; s++)
			{
				__syncthreads();
				fetch_b(rb[s & 1]);
				multiply(s & 1);
				stash((s + 1) & 1, ra[(s + 1) % STEPS], rb[(s + 1) & 1]);
				fetch_a(ra[(s + 1) % STEPS]);
			}
			/* buffer 1 was multiplied last and is refilled only after the next barrier of the loop above: the accumulators
			 * leave through it while buffer 0 already holds step 0 of the next tile */
			const int64_t p0 = static_cast<int64_t>(pb) * BLOCK_M;
			typename Epi::template ColumnsT<W> columns;
			if (k < g.K)
				Epi::pick_columns(table, k, columns);
			drain_tile<TE, 2, 2, W>(lds + 2 * LDS_TILE, acc, [&](int r, const typename Epi::scalar_t (&v)[W], int) __attribute__((always_inline))
			{
				const int64_t p = p0 + r;
				if (p < g.pixels && k < g.K)
					epi.template store_at<ACT_SIMPLE, true, W>(p * g.K + k, k, v, columns);
			});
		}
	}
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
		if (static_cast<size_t>(s.K) * sizeof(typename Epi::template ColumnsT<1>) > static_cast<size_t>(TABLE_BYTES))
			return false;
		const int64_t pixels = static_cast<int64_t>(s.N) * s.H * s.W;
		const int64_t pixel_blocks = (pixels + BLOCK_M - 1) / BLOCK_M, filter_blocks = (static_cast<int64_t>(s.K) + BLOCK_N - 1) / BLOCK_N;
		const int64_t tiles = pixel_blocks * filter_blocks;
		if (pixels >= (1ll << 31) - BLOCK_M || tiles >= (1ll << 31) - 1024)
			return false;
		PointGeom g;
		g.pixels = static_cast<int>(pixels);
		g.K = s.K;
		g.row_bytes = static_cast<unsigned int>(s.C) * static_cast<unsigned int>(sizeof(TE));
		const int steps = static_cast<int>((g.row_bytes + STEP_BYTES - 1) / STEP_BYTES);
		if (steps > 4)
			return false; /* a register set of x per step: longer rows stay with the gather kernel, whose k loop is long enough */
		g.filter_blocks = static_cast<int>(filter_blocks);
		g.tiles = static_cast<int>(tiles);
		/* two workgroups per compute unit stay resident; with fewer tiles than that every workgroup has one tile */
		int device = 0, units = 256;
		if (hipGetDevice(&device) == hipSuccess)
			(void) hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device);
		const int resident = 2 * (units > 0 ? units : 256);
		const dim3 grid(static_cast<unsigned int>(tiles < resident ? tiles : resident));
		if (steps <= 2)
			hipLaunchKernelGGL((k_conv_pointwise<TE, Epi, 2>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		else
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
