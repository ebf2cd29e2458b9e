/*
 * conv_tile.hip -- implicit-GEMM convolution for stride-1 filters that keeps an image tile resident in LDS.
 *
 * The general implicit-GEMM kernel (conv_implicit_gemm.hip) re-fetches every input pixel once per filter tap from L2: for
 * a 3x3 filter that is 9x the input volume plus the weights once per 128 output pixels, and on MI355X this L2 -> CU traffic,
 * not the matrix cores, bounds it.  This kernel removes most of that traffic:
 *
 *   - a workgroup owns TH x TW <= 256 output pixels of ONE image (the whole image when it is 15 x 15) and 64 filters;
 *   - for each 128-byte slice of input channels it loads the (TH+R-1) x (TW+S-1) input halo ONCE into LDS (pixels outside
 *     the image come back as zeros from the buffer load) and then walks the R*S taps, reading the A operand of tap (i, j)
 *     straight from the halo at a per-tap uniform offset: the input is read from L2 about once per slice, not R*S times;
 *   - only the weights stream: 64 filters x 128 bytes per step, fetched three steps ahead into registers (three sets) and
 *     double buffered in LDS;
 *   - the halo of the next channel slice is fetched during the third tap of the current one and held in registers.
 * Four wavefronts stack in M (64 pixels x 64 filters each, 2 x 2 MFMA tiles of 32 x 32); 72 KB of LDS and <= 256 registers
 * let two workgroups share a CU.  k order is (channel slice, tap), which sums the same products as (tap, channel).
 *
 * The 256 rows of the workgroup's GEMM tile are NOT the TH x TW output pixels in raster order: row q stands for halo
 * position q (halo rows are HW = TW + S - 1 pixels long), so S - 1 rows at the end of every tile row compute values that
 * nobody stores.  In exchange the A operand of tap (i, j) for row q is halo pixel q + i * HW + j: the 32 rows of an MFMA
 * tile always read 32 CONSECUTIVE halo pixels, whatever the tap, and with the 144-byte pixel pitch that is free of LDS
 * bank conflicts (raster order breaks the run at every tile-row end), and no per-row division is needed for the addresses.
 * The general instance (filters other than 3 x 3) may be launched in raster ("dense") order instead, and with an LDS layout
 * that holds a larger halo at one workgroup per compute unit: a wide tile under a large filter does not fit 256 rows in halo
 * order, and fewer, fuller tiles then outweigh the conflicts (see TileLds and choose_tile).
 *
 * Epilogue: the accumulators leave through LDS so that a work-item stores 16 bytes of consecutive filters of one pixel with a
 * streaming store; a table in LDS maps GEMM rows to output pixels; the residual z of the rows a work-item will store is fetched
 * during the last channel slice, not between the stores (where possible aliasing of y and z would serialise the loads).
 * Workgroups are numbered so that the tiles of an image, which share halo pixels, run on one XCD.
 */
#include "conv_tile.hpp"
#include "mfma_core.hpp"
#include "persistent_gemm.hpp"
#include <type_traits>

/* Instrumentation, compiled in with -DCONV_TILE_STAMPS only: wavefront 0 of every workgroup records the 100 MHz wall clock at
 * the phase boundaries of the kernel (start, arguments read, requests out, halo in LDS, first MFMA, loop end, epilogue end), and
 * avhip_debug_stamps() copies the records of the last launch to the host.  The phase timings quoted for this kernel come from it. */
#ifdef CONV_TILE_STAMPS
__device__ unsigned long long g_stamps[4096 * 8];
#define STAMP(i) do { if (threadIdx.x == 0) g_stamps[(blockIdx.x % 4096) * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
extern "C" __attribute__((visibility("default"))) int avhip_debug_stamps(void *out)
{
	return static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_stamps), sizeof(g_stamps)));
}
#else
#define STAMP(i) do { } while (0)
#endif

namespace
{
	using namespace avhip;

	constexpr int TILE_M = 256; /* output pixels per workgroup */
	constexpr int TILE_N = 64; /* output filters per workgroup */
	constexpr int PIXEL_PITCH = STEP_BYTES + 16; /* LDS bytes per halo pixel: 128 of channels + 16 of bank stagger */
	constexpr int FILTER_TILE = TILE_N * LDS_ROW;
	constexpr int FILTER_RING = 3; /* filter tiles in LDS: two for the general k loop, a ring of three for the unrolled 3x3 one */
	constexpr int FILTER_FETCHES = TILE_N * STEP_CHUNKS / 256;
	/* LDS of a workgroup, by the halo pixels it can hold: [halo | filter ring | row table].  300 pixels (the 17 x 17 halo of a
	 * 15 x 15 image) leave room for two workgroups per compute unit; 448 (a 12 x 36 halo: 8 x 32 outputs under a 5 x 5 filter)
	 * fill a compute unit with one. */
	constexpr int HALO_SMALL = 300, HALO_BIG = 448;
	template<int HMAX> struct TileLds
	{
		static constexpr int halo_bytes = HMAX * PIXEL_PITCH;
		static constexpr int row_table = halo_bytes + FILTER_RING * FILTER_TILE; /* GEMM row -> offset of its output pixel in the image, -1 if not stored */
		static constexpr int bytes = row_table + TILE_M * 4;
		static constexpr int halo_fetches = (HMAX * STEP_CHUNKS + 255) / 256; /* 16-byte chunks of the halo per work-item */
		static constexpr int pixels = (halo_bytes + 2 * FILTER_TILE) / PIXEL_PITCH; /* what a read at a halo-order row may reach */
	};
	static_assert(4 * PrivateDrainRows<2, 4>::bytes <= TileLds<HALO_SMALL>::row_table, "the drain buffers of the four wavefronts reuse the operand buffers");

	struct TileGeom
	{
		int H, W, C, K, R, S, Ho, Wo, pad_h, pad_w, flip;
		int TH, TW; /* output tile */
		int HH, HW; /* halo = (TH + R - 1) x (TW + S - 1) */
		unsigned int hw_magic; /* 2^20 / HW + 1: (v * hw_magic) >> 20 == v / HW while v * HW < 2^20 */
		int row_pitch; /* GEMM row r is output pixel (r / row_pitch, r % row_pitch) of the tile: HW (halo order) or TW (dense) */
		unsigned int row_magic; /* 2^20 / row_pitch + 1 */
		int tiles_h, tiles_w;
		int slices; /* 128-byte channel slices */
		int images;
		int filter_blocks; /* blocks of TILE_N filters */
		int filter_shift; /* log2(filter_blocks) when that is a power of two, else -1 */
		int filter_fastest; /* numbering of the workgroups, see the kernel */
	};

	/* FS = 3: the filter is 3 x 3 and the k loop is written out tap by tap (see the second half of the kernel); FS = 0: any
	 * filter, general loop. */
	template<typename TE, typename Epi, int FS, int HMAX = HALO_SMALL>
	__global__ __launch_bounds__(256, HMAX > HALO_SMALL ? 1 : 2) void k_conv_tile(const TE *__restrict__ x, const TE *__restrict__ w, TileGeom g, Epi epi)
	{
		constexpr int HALO_MAX = HMAX;
		constexpr int HALO_BYTES = TileLds<HMAX>::halo_bytes;
		constexpr int ROW_TABLE = TileLds<HMAX>::row_table;
		constexpr int TILE_LDS = TileLds<HMAX>::bytes;
		constexpr int HALO_FETCHES = TileLds<HMAX>::halo_fetches;
		STAMP(0);
		epi.pin();
		keep_in_sgpr(g.TW);
		keep_in_sgpr(g.TH);
		keep_in_sgpr(g.Ho);
		keep_in_sgpr(g.Wo);
		keep_in_sgpr(g.K);
		STAMP(6);
		__shared__ __attribute__((aligned(16))) char lds[TILE_LDS];
		char *halo = lds;
		char *filt = lds + HALO_BYTES;
		constexpr int E = 16 / sizeof(TE);
		constexpr int KE = STEP_BYTES / sizeof(TE);
		constexpr unsigned int SZ = sizeof(TE);
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int part = tid % STEP_CHUNKS;
		const int chunk_channel = part * E;

		/* Everything up to the first halo request is latency the matrix cores sit through: no division on that path when the
		 * tile is the whole image, and divisions by the halo width as a multiplication (hw_magic). */
		/* One-dimensional grid over (tile, filter block), tiles XCD-contiguous (the tiles of an image share halo pixels: one L2).
		 * Grids of several rounds number the filter block fastest: the workgroups that read the same halo are then dispatched next
		 * to each other and the halo comes from memory once, from L2 afterwards (measured 3-6 % on 56 x 56 x 256 layers).  Grids
		 * that are resident at once keep the tiles fastest: there both filter blocks of a tile land on one compute unit (measured
		 * 5 % better on 20 x 20 x 128 in bf16 than the other order). */
		unsigned int filter_block, tile_number;
		if (g.filter_fastest)
		{
			const unsigned int work = xcd_block(blockIdx.x, gridDim.x);
			if (g.filter_shift >= 0)
			{
				filter_block = work & ((1u << g.filter_shift) - 1u);
				tile_number = work >> g.filter_shift;
			}
			else
			{
				tile_number = work / static_cast<unsigned int>(g.filter_blocks);
				filter_block = work - tile_number * g.filter_blocks;
			}
		}
		else
		{
			const unsigned int tiles = gridDim.x / static_cast<unsigned int>(g.filter_blocks);
			filter_block = g.filter_blocks == 1 ? 0u : blockIdx.x / tiles;
			tile_number = xcd_block(blockIdx.x - filter_block * tiles, tiles);
		}
		int b = static_cast<int>(tile_number);
		int tw = 0, th = 0, n = b;
		if (g.tiles_w * g.tiles_h != 1)
		{
			tw = b % g.tiles_w;
			b /= g.tiles_w;
			th = b % g.tiles_h;
			n = b / g.tiles_h;
		}
		const int oh0 = th * g.TH, ow0 = tw * g.TW;
		const int k0 = static_cast<int>(filter_block) * TILE_N;
		constexpr int W = Epi::wide; /* filters per work-item in the epilogue: one 16-byte store each */
		const int kcol = k0 + drain_column<1, W>();
		typename Epi::template ColumnsT<W> columns;

		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, static_cast<unsigned int>(g.images) * g.H * g.W * g.C * SZ);
		const __amdgpu_buffer_rsrc_t rw = make_buffer(w, static_cast<unsigned int>(g.K) * g.R * g.S * g.C * SZ);

		const int halo_dst = (tid / STEP_CHUNKS) * PIXEL_PITCH + part * 16;
		unsigned int filt_src[FILTER_FETCHES];
#pragma unroll
		for (int f = 0; f < FILTER_FETCHES; f++)
		{
			const int k = k0 + tid / STEP_CHUNKS + f * (256 / STEP_CHUNKS);
			filt_src[f] = k < g.K ? static_cast<unsigned int>(k * g.R * g.S * g.C + chunk_channel) * SZ : OUT_OF_RANGE;
		}
		const int filt_dst = (tid / STEP_CHUNKS) * LDS_ROW + part * 16;
		unsigned int halo_src[HALO_FETCHES];
		const int halo_pixels = g.HH * g.HW;
		const int taps = g.R * g.S;
		const int total = g.slices * taps;
		const int prefetch_tap = taps > 2 ? 2 : taps - 1;

		/* fetch side: runs three steps ahead of the MFMAs.  The first requests go out before anything else is computed: the
		 * addresses of the filters are the cheapest to form, the halo's follow, and the bookkeeping that needs no memory (row
		 * table, accumulators) is done while they travel. */
		int f_slice = 0, f_tap = 0;
		auto fetch_filters = [&](uint4 (&r)[FILTER_FETCHES]) __attribute__((always_inline))
		{
			const unsigned int k_bytes = static_cast<unsigned int>(f_tap * g.C) * SZ + static_cast<unsigned int>(f_slice) * STEP_BYTES;
			const bool exists = (f_slice * KE + chunk_channel < g.C) & (f_slice < g.slices);
#pragma unroll
			for (int f = 0; f < FILTER_FETCHES; f++)
				r[f] = buffer_fetch(rw, exists ? filt_src[f] + k_bytes : OUT_OF_RANGE);
			if (++f_tap == taps)
			{
				f_tap = 0;
				f_slice++;
			}
		};
		auto stash_filters = [&](int buffer, const uint4 (&r)[FILTER_FETCHES]) __attribute__((always_inline))
		{
#pragma unroll
			for (int f = 0; f < FILTER_FETCHES; f++)
				*reinterpret_cast<uint4*>(filt + buffer * FILTER_TILE + filt_dst + f * (256 / STEP_CHUNKS) * LDS_ROW) = r[f];
		};
		auto fetch_halo = [&](int slice, uint4 (&r)[HALO_FETCHES]) __attribute__((always_inline))
		{
			const bool exists = slice * KE + chunk_channel < g.C;
#pragma unroll
			for (int f = 0; f < HALO_FETCHES; f++)
				r[f] = buffer_fetch(rx, exists ? halo_src[f] + static_cast<unsigned int>(slice) * STEP_BYTES : OUT_OF_RANGE);
		};
		auto stash_halo = [&](const uint4 (&r)[HALO_FETCHES]) __attribute__((always_inline))
		{
#pragma unroll
			for (int f = 0; f < HALO_FETCHES; f++)
				if (tid / STEP_CHUNKS + f * (256 / STEP_CHUNKS) < HALO_MAX)
					*reinterpret_cast<uint4*>(halo + halo_dst + f * (256 / STEP_CHUNKS) * PIXEL_PITCH) = r[f];
		};
		uint4 hr[HALO_FETCHES];
		uint4 fr[3][FILTER_FETCHES];
		fetch_filters(fr[0]);
		fetch_filters(fr[1]);
		fetch_filters(fr[2]);
		STAMP(7);
		/* where this work-item's halo chunks come from (slice 0).  Integer division by a run-time divisor costs about thirty
		 * instructions and a 32-bit multiply four issue slots: the work-item divides once and then walks, position and byte
		 * offset alike (the offset of a pixel outside the image is never used; inside the image it is below 2 GiB and the
		 * additions are exact modulo 2^32). */
		{
			/* Ten independent address computations, none waiting for another and none behind a branch: vector instructions of a
			 * wavefront issue every fourth clock and two wavefronts share a SIMD, so every instruction here is eight clocks of
			 * the time before the first MFMA.  The halo position divides by the halo width with a 24-bit multiplication. */
			constexpr int STRIDE = 256 / STEP_CHUNKS; /* halo pixels between two fetches of a work-item */
			const unsigned int pixel_bytes = static_cast<unsigned int>(g.C) * SZ;
			const bool first_slice_exists = chunk_channel < g.C;
			const unsigned int line_bytes = static_cast<unsigned int>(g.W) * pixel_bytes;
			const int ih0 = oh0 + g.pad_h, iw0 = ow0 + g.pad_w;
			/* byte offset of halo pixel (0, 0), which may lie outside the image: the sum with a pixel's (hy, hx) part is exact
			 * modulo 2^32 and only used when the pixel is inside */
			const unsigned int base = (static_cast<unsigned int>(n) * static_cast<unsigned int>(g.H) + static_cast<unsigned int>(ih0)) * line_bytes
					+ static_cast<unsigned int>(iw0) * pixel_bytes + static_cast<unsigned int>(chunk_channel) * SZ;
#pragma unroll
			for (int f = 0; f < HALO_FETCHES; f++)
			{
				const unsigned int h = static_cast<unsigned int>(tid / STEP_CHUNKS + f * STRIDE);
				const unsigned int hy = __umul24(h, g.hw_magic) >> 20; /* h < 512, hw_magic <= 2^20 / 3 + 1 */
				const unsigned int hx = h - __umul24(hy, static_cast<unsigned int>(g.HW));
				const bool inside = (h < static_cast<unsigned int>(halo_pixels)) & (static_cast<unsigned int>(ih0) + hy < static_cast<unsigned int>(g.H))
						& (static_cast<unsigned int>(iw0) + hx < static_cast<unsigned int>(g.W));
				/* both factors of either product are below 2^24 (the launcher checks the row and pixel sizes) */
				const unsigned int offset = base + __umul24(hy, line_bytes) + __umul24(hx, pixel_bytes);
				halo_src[f] = inside ? offset : OUT_OF_RANGE;
				hr[f] = buffer_fetch(rx, first_slice_exists ? halo_src[f] : OUT_OF_RANGE); /* slice 0 goes out as soon as its address exists */
				__builtin_amdgcn_sched_barrier(0); /* ... and the scheduler may not collect the requests behind all the address arithmetic */
			}
		}
		STAMP(4);
		epi.request_columns(kcol, columns); /* needed in the epilogue only: behind everything the first MFMA waits for, and nothing waits for it */
		int *row_table = reinterpret_cast<int*>(lds + ROW_TABLE);
		{
			/* GEMM row -> offset of its output pixel inside the image of y, in elements; -1 for rows that are not stored */
			/* (the written-out 3 x 3 instance is launched in halo order only and spends nothing on the other one) */
			const unsigned int pitch = FS != 3 ? static_cast<unsigned int>(g.row_pitch) : static_cast<unsigned int>(g.HW), magic = FS != 3 ? g.row_magic : g.hw_magic;
			const int py = static_cast<int>((static_cast<unsigned int>(tid) * magic) >> 20), px = tid - py * static_cast<int>(pitch);
			const int oh = oh0 + py, ow = ow0 + px;
			row_table[tid] = (py < g.TH && px < g.TW && oh < g.Ho && ow < g.Wo) ? (oh * g.Wo + ow) * g.K : -1; /* times K here, once, not in every use */
		}

		/* MFMA operand addresses: lane l supplies row (l % 32) of a 32-row tile and k-chunk (l / 32) */
		int a_off[2];
		const int b_off = (lane & 31) * LDS_ROW + (lane >> 5) * 16;

		typename Mma<TE>::acc_t acc[2][2];
		if constexpr (FS == 0)
		{
#pragma unroll
			for (int i = 0; i < 2; i++)
#pragma unroll
				for (int j = 0; j < 2; j++)
#pragma unroll
					for (int v = 0; v < 16; v++)
						acc[i][j][v] = 0;
		}

		/* compute side */
		int c_slice = 0, c_i = 0, c_j = 0;
		auto multiply = [&](int buffer) __attribute__((always_inline))
		{
			const int i = g.flip ? g.R - 1 - c_i : c_i;
			const int j = g.flip ? g.S - 1 - c_j : c_j;
			const char *sa = halo + (i * g.HW + j) * PIXEL_PITCH;
			const char *sb = filt + buffer * FILTER_TILE + b_off;
			constexpr int SLABS = STEP_BYTES / 32;
			Chunk a[2][2], bq[2][2];
			auto read = [&](int slab, Chunk (&ra_)[2], Chunk (&rb_)[2]) __attribute__((always_inline))
			{
#pragma unroll
				for (int t = 0; t < 2; t++)
				{
					ra_[t].u = *reinterpret_cast<const uint4*>(sa + a_off[t] + slab * 32);
					rb_[t].u = *reinterpret_cast<const uint4*>(sb + t * 32 * LDS_ROW + slab * 32);
				}
			};
			read(0, a[0], bq[0]);
#pragma unroll
			for (int slab = 0; slab < SLABS; slab++)
			{
				if (slab + 1 < SLABS)
					read(slab + 1, a[(slab + 1) & 1], bq[(slab + 1) & 1]);
				/* a wavefront with operands in hand goes ahead of one that is still issuing loads */
				burst_priority(slab);
#pragma unroll
				for (int tm = 0; tm < 2; tm++)
#pragma unroll
					for (int tn = 0; tn < 2; tn++)
						Mma<TE>::run(a[slab & 1][tm], bq[slab & 1][tn], acc[tm][tn]);
				if (slab + 1 == SLABS)
					__builtin_amdgcn_s_setprio(0);
			}
			/* instruction order within the step: after the first slab's reads, one LDS read behind every MFMA, so that reads
			 * of the next slab trickle out under the matrix pipeline instead of in a burst between two groups of MFMAs */
#pragma unroll
			for (int i = 0; i < 4 * (SLABS - 1); i++)
			{
				__builtin_amdgcn_sched_group_barrier(0x008, 1, 0); /* one MFMA */
				__builtin_amdgcn_sched_group_barrier(0x100, 1, 0); /* one LDS read */
			}
		};

		/* the halo pixel under tap (0, 0) of this work-item's GEMM rows.  In halo order (row pitch = halo width) that is the row
		 * number itself and rows between the tile's lines are computed and dropped; in dense order (row pitch = tile width: every
		 * row is a pixel, for tiles whose lines in halo order would not fit 256 rows) rows past the tile read pixel 0 */
#pragma unroll
		for (int tm = 0; tm < 2; tm++)
			a_off[tm] = (wave * 64 + tm * 32 + (lane & 31)) * PIXEL_PITCH + (lane >> 5) * 16;
		if (FS != 3 && g.row_pitch != g.HW) /* (uniform) */
		{
#pragma unroll
			for (int tm = 0; tm < 2; tm++)
			{
				const int r = wave * 64 + tm * 32 + (lane & 31);
				const int py = static_cast<int>((static_cast<unsigned int>(r) * g.row_magic) >> 20), px = r - py * g.row_pitch;
				a_off[tm] = (py < g.TH ? py * g.HW + px : 0) * PIXEL_PITCH + (lane >> 5) * 16;
			}
		}
		stash_halo(hr);
		stash_filters(0, fr[0]);
		STAMP(5);

		/* The residual of every row this work-item will store is requested during the last channel slice: its latency and its
		 * HBM traffic run under the MFMAs of that slice instead of in the epilogue, and the registers are held for half the
		 * loop only. */
		typedef PrivateDrainRows<2, W> Rows;
		const int64_t image_base = static_cast<int64_t>(n) * g.Ho * g.Wo * g.K + kcol; /* element index of (image n, pixel 0, filter kcol); one image of y is below 2^31 elements (checked by the launcher) */
		/* (16-bit and int8 tensors only: sixteen rows of four fp32 values are 64 registers, which the fp32 instance does not
		 * have; it loads its residual row by row in the epilogue) */
		constexpr bool RESIDUAL_AHEAD = sizeof(TE) < 4;
		typename Epi::template Residual<W> residual[RESIDUAL_AHEAD ? Rows::slots : 1];
		auto fetch_residual = [&]() __attribute__((always_inline))
		{
			if (!RESIDUAL_AHEAD)
				return;
#pragma unroll
			for (int slot = 0; slot < Rows::slots; slot++)
			{
				const int e = row_table[Rows::row(slot)];
				if (e >= 0 && kcol < g.K)
					epi.load_residual(image_base + e, residual[RESIDUAL_AHEAD ? slot : 0]);
			}
		};

		/* One step = one tap of one channel slice.  The filters of step t are requested at step t - 3 into register set t % 3,
		 * go to LDS buffer t % 2 at the end of step t - 1 and are multiplied at step t: a load from L2 has two full steps of
		 * MFMAs to arrive.  Six steps per trip keep the set and buffer indices compile-time constants; fetches past the last
		 * step return zeros and steps past it are not multiplied. */
		auto step = [&](int s, int buffer, uint4 (&mine)[FILTER_FETCHES], uint4 (&next)[FILTER_FETCHES]) __attribute__((always_inline))
		{
			__syncthreads(); /* filters of step s and the current halo are visible; everyone is done with step s - 1 */
			fetch_filters(mine); /* step s + 3: this set held step s, which went to LDS during step s - 1 */
			/* the halo of the next channel slice is requested early in the current one (its registers are free from the
			 * moment the current halo went to LDS), so that its latency is spent under several taps of MFMAs */
			const bool prefetch_now = c_i * g.S + c_j == prefetch_tap;
			const bool more_slices = c_slice + 1 < g.slices;
			if (prefetch_now & more_slices)
				fetch_halo(c_slice + 1, hr);
			if (prefetch_now & !more_slices)
				fetch_residual(); /* after the barrier above, so the row table is complete */
			if (s < total)
				multiply(buffer);
			stash_filters(buffer ^ 1, next); /* step s + 1 */
			if (++c_j == g.S)
			{
				c_j = 0;
				if (++c_i == g.R)
				{
					c_i = 0;
					c_slice++;
					if (c_slice < g.slices)
					{
						__syncthreads(); /* nobody reads the old halo any more */
						stash_halo(hr);
					}
				}
			}
		};
		if constexpr (FS > 0)
		{
			/*
			 * 3 x 3 filters: the k loop written out, one channel slice = nine steps with nothing conditional inside.
			 *
			 * Why: loads return in order and the compiler counts them statically.  In the general loop below the halo and
			 * residual prefetches sit behind run-time conditions, so every later wait for a filter load has to assume they
			 * were not issued and ends up waiting for them as well: a whole HBM latency, twice per tile.  Written out, every
			 * wait names exactly the loads it needs.  The filters go through a ring of three LDS tiles (tap % 3; nine taps
			 * keep the phase) instead of two, which makes the tile of step t + 1 visible during step t: the operands of the
			 * first 32-byte slab of the next step are read while the last MFMAs of the current one run, so the LDS latency
			 * after each barrier is off the critical path too.
			 *
			 * Filters of step t: requested at the top of step t - 3 into register set t % 3, written to ring[t % 3] at the
			 * end of step t - 2 (everyone has passed the barrier of step t - 2, so nobody reads step t - 3's tile any more),
			 * visible from the barrier of step t - 1.
			 */
			constexpr int TAPS = FS * FS;
			constexpr int SLABS = STEP_BYTES / 32;
			constexpr int PREFETCH_TAP = 2;
			/* (5 x 5: 25 taps shift the ring phase from one slice to the next, so that instance is launched for layers of a single
			 * channel slice only) */
			static_assert(TAPS % FILTER_RING == 0 || FS == 5, "the ring phase must be the same in every channel slice");
			stash_filters(1, fr[1]);
			const int row_pitch = g.HW * PIXEL_PITCH;
			const int flip_base = g.flip ? (FS - 1) * (row_pitch + PIXEL_PITCH) : 0;
			const int flip_sign = g.flip ? -1 : 1;
			Chunk a[2][2], bq[2][2]; /* operands of two consecutive slabs; they live across steps */
			auto read = [&](int tap, int slab, Chunk (&ra_)[2], Chunk (&rb_)[2]) __attribute__((always_inline))
			{
				const char *sa = halo + flip_base + flip_sign * ((tap / FS) * row_pitch + (tap % FS) * PIXEL_PITCH);
				const char *sb = filt + (tap % FILTER_RING) * FILTER_TILE + b_off;
#pragma unroll
				for (int t = 0; t < 2; t++)
				{
					ra_[t].u = *reinterpret_cast<const uint4*>(sa + a_off[t] + slab * 32);
					rb_[t].u = *reinterpret_cast<const uint4*>(sb + t * 32 * LDS_ROW + slab * 32);
				}
			};
			auto fetch_filters_at = [&](int slice, int tap, uint4 (&r)[FILTER_FETCHES]) __attribute__((always_inline))
			{
				const int sl = tap >= TAPS ? slice + 1 : slice, tp = tap >= TAPS ? tap - TAPS : tap;
				const unsigned int k_bytes = static_cast<unsigned int>(tp * g.C) * SZ + static_cast<unsigned int>(sl) * STEP_BYTES;
				const bool exists = sl * KE + chunk_channel < g.C; /* false for every slice past the last */
#pragma unroll
				for (int f = 0; f < FILTER_FETCHES; f++)
					r[f] = buffer_fetch(rw, exists ? filt_src[f] + k_bytes : OUT_OF_RANGE);
			};
			/* the residual through a buffer load: rows that are not stored ask for an out-of-range offset instead of being
			 * skipped, so the number of loads in flight does not depend on the data */
			constexpr bool RESIDUAL_BUFFER = RESIDUAL_AHEAD && sizeof(TE) == 2;
			__amdgpu_buffer_rsrc_t rz = make_buffer(nullptr, 0);
			if constexpr (RESIDUAL_BUFFER)
				if (epi.z != nullptr)
					rz = make_buffer(epi.z + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K, static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ);
			auto fetch_residual_rows = [&]() __attribute__((always_inline))
			{
				if constexpr (RESIDUAL_BUFFER)
				{
#pragma unroll
					for (int slot = 0; slot < Rows::slots; slot++)
					{
						const int e = row_table[Rows::row(slot)];
						union
						{
							uint4 u;
							decltype(residual[0].raw) p;
						} cast;
						cast.u = buffer_fetch<2>(rz, (e >= 0 && kcol < g.K) ? static_cast<unsigned int>(e + kcol) * SZ : OUT_OF_RANGE);
						residual[slot].raw = cast.p;
					}
				}
			};
			/* FIRST: the very first MFMA of each accumulator starts from the constant zero, so the 64 accumulator registers are
			 * not cleared (64 moves per wavefront, right on the way to the first MFMA: they share registers with the staged
			 * halo and cannot be hoisted above the loads' arrival) */
			auto slice_steps = [&](int slice, auto is_first, auto is_last) __attribute__((always_inline))
			{
				constexpr bool FIRST = decltype(is_first)::value;
				constexpr bool LAST = decltype(is_last)::value;
#pragma unroll
				for (int tap = 0; tap < TAPS; tap++)
				{
					__syncthreads(); /* ring[(tap + 1) % 3] and, at tap 0, the halo are visible; everyone is done with the step before */
#ifdef CONV_TILE_STAMPS
					if (tap == 0 && slice == 0)
						STAMP(1);
#endif
					if (tap == 0)
						read(0, 0, a[0], bq[0]); /* the halo changed under the barrier above: nothing could be read ahead */
#pragma unroll
					for (int slab = 0; slab < SLABS; slab++)
					{
						if (slab + 1 < SLABS)
							read(tap, slab + 1, a[(slab + 1) & 1], bq[(slab + 1) & 1]);
						else if (tap + 1 < TAPS)
							read(tap + 1, 0, a[0], bq[0]);
						burst_priority(slab);
#pragma unroll
						for (int tm = 0; tm < 2; tm++)
#pragma unroll
							for (int tn = 0; tn < 2; tn++)
							{
								if (FIRST && tap == 0 && slab == 0)
									Mma<TE>::start(a[slab & 1][tm], bq[slab & 1][tn], acc[tm][tn]);
								else
									Mma<TE>::run(a[slab & 1][tm], bq[slab & 1][tn], acc[tm][tn]);
							}
						if (slab + 1 == SLABS)
							__builtin_amdgcn_s_setprio(0);
					}
					/* one LDS read behind every MFMA */
#pragma unroll
					for (int i = 0; i < 4 * (SLABS - 1) + (tap + 1 < TAPS ? 4 : 0); i++)
					{
						__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
						__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
					}
					/* requests for later steps cost only issue slots: behind the MFMAs of this one */
					fetch_filters_at(slice, tap + 3, fr[tap % 3]);
					if (tap == PREFETCH_TAP)
					{
						if constexpr (LAST)
							fetch_residual_rows();
						else
							fetch_halo(slice + 1, hr);
					}
					stash_filters((tap + 2) % FILTER_RING, fr[(tap + 2) % FILTER_RING]);
				}
				if constexpr (!LAST)
				{
					__syncthreads(); /* nobody reads the old halo any more */
					stash_halo(hr);
				}
			};
			if (g.slices == 1 || TAPS % FILTER_RING != 0)
				slice_steps(0, std::true_type(), std::true_type());
			else
			{
				slice_steps(0, std::true_type(), std::false_type());
				for (int slice = 1; slice + 1 < g.slices; slice++)
					slice_steps(slice, std::false_type(), std::false_type());
				slice_steps(g.slices - 1, std::false_type(), std::true_type());
			}
		}
		else
		for (int s = 0; s < total; s += 6)
		{
			step(s, 0, fr[0], fr[1]);
			step(s + 1, 1, fr[1], fr[2]);
			step(s + 2, 0, fr[2], fr[0]);
			step(s + 3, 1, fr[0], fr[1]);
			step(s + 4, 0, fr[1], fr[2]);
			step(s + 5, 1, fr[2], fr[0]);
		}

		STAMP(2);
		epi.finish_columns(columns);
		if constexpr (std::is_same<Epi, FloatEpilogue<TE>>::value && sizeof(TE) == 2)
		{
			/* 16-bit tensors with beta = 0: the epilogue without a single branch.  Which of the four forms (ReLU, residual) is
			 * decided once, rows that are not stored go to an out-of-range offset of a buffer over this image of y, and the
			 * eight runs of a work-item can be scheduled into each other. */
			/* (an image of y must stay below the out-of-range marker, or a row that is not stored would land inside it) */
			if (epi.beta == 0.0f && static_cast<int64_t>(g.Ho) * g.Wo * g.K * SZ < (1ll << 31))
			{
				const __amdgpu_buffer_rsrc_t ry = make_buffer(epi.y + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K, static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ);
				auto drain = [&](auto relu, auto has_z) __attribute__((always_inline))
				{
					drain_tile_private<TE, 2, W>(lds, acc, [&](int row, const float (&v)[W], int slot) __attribute__((always_inline))
					{
						const int e = row_table[row];
						const unsigned int offset = (e >= 0 && kcol < g.K) ? static_cast<unsigned int>(e + kcol) * SZ : OUT_OF_RANGE;
						epi.template store_fast<decltype(relu)::value, decltype(has_z)::value, W>(v, columns, residual[slot], [&](auto words) __attribute__((always_inline))
						{
							buffer_put<STORE_STREAM_THROUGH>(ry, offset, words);
						});
					});
				};
				const bool relu = epi.activation == ACT_RELU, has_z = epi.z != nullptr;
				if (relu && has_z)
					drain(std::true_type(), std::true_type());
				else if (relu)
					drain(std::true_type(), std::false_type());
				else if (has_z)
					drain(std::false_type(), std::true_type());
				else
					drain(std::false_type(), std::false_type());
				STAMP(3);
				return;
			}
		}
		drain_tile_private<TE, 2, W>(lds, acc, [&](int row, const typename Epi::scalar_t (&v)[W], int slot) __attribute__((always_inline))
		{
			const int e = row_table[row];
			if (e >= 0 && kcol < g.K)
				epi.template store_at<ACT_SIMPLE, true, W>(image_base + e, kcol, v, columns, RESIDUAL_AHEAD ? &residual[slot] : nullptr);
		});
		STAMP(3);
	}

	template<typename TE> bool columns_aligned(const FloatEpilogue<TE>&)
	{
		return true;
	}
	/* a workgroup of this kernel stores TILE_N = 64 filters of a pixel: int8 results are half a cache line */
	template<typename TE> FloatEpilogue<TE> for_partial_lines(const FloatEpilogue<TE> &epi)
	{
		return epi;
	}
	template<int MODE> Int8Epilogue<MODE> for_partial_lines(const Int8Epilogue<MODE> &epi)
	{
		Int8Epilogue<MODE> e = epi;
		e.through = true;
		return e;
	}
	template<int MODE> bool columns_aligned(const Int8Epilogue<MODE> &epi)
	{
		return aligned_to(epi.scale, 16);
	}

	/* Picks the output tile for a halo capacity: as few tiles per image as possible such that the tile's rows fit the 256 GEMM
	 * rows and its halo fits LDS.  Rows in halo order (the tile's lines at the pitch of the halo: a tap is one constant shift of
	 * consecutive LDS pixels, conflict-free reads; the reads of the never-stored rows must stay inside the kernel's LDS) are
	 * preferred; dense order (every row a pixel) takes over where it needs fewer tiles, which is the case for wide tiles under
	 * large filters. */
	struct TileChoice
	{
		int th, tw, dense, tiles;
	};
	TileChoice choose_tile(const avhipConvShape &s, int halo_max, int lds_pixels, bool allow_dense)
	{
		TileChoice best = { 0, 0, 0, 0 };
		int best_halo = 0;
		for (int dense = 0; dense < (allow_dense ? 2 : 1); dense++)
			for (int tw = 1; tw <= s.Wo && tw <= TILE_M; tw++)
				for (int th = 1; th <= s.Ho; th++)
				{
					const int hw = tw + s.S - 1;
					const int rows = dense ? th * tw : (th - 1) * hw + tw;
					const int halo = (th + s.R - 1) * hw;
					if (rows > TILE_M)
						break;
					if (halo > halo_max || (!dense && TILE_M + (s.R - 1) * hw + s.S > lds_pixels))
						continue;
					const int tiles = ((s.Ho + th - 1) / th) * ((s.Wo + tw - 1) / tw);
					if (best.tiles == 0 || tiles < best.tiles || (tiles == best.tiles && dense == best.dense && halo < best_halo))
					{
						best = { th, tw, dense, tiles };
						best_halo = halo;
					}
				}
		return best;
	}
}

namespace avhip
{
	template<typename TE, typename Epi>
	bool conv_tile_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &caller_epi)
	{
		const Epi epi = for_partial_lines(caller_epi);
		if (s.stride_h != 1 || s.stride_w != 1 || s.dil_h != 1 || s.dil_w != 1)
			return false;
		/* the kernel stores whole runs of Epi::wide filters with one 16-byte instruction */
		if (!epi.vec || s.K % Epi::wide != 0 || !aligned_to(epi.y, 16) || (epi.z != nullptr && !aligned_to(epi.z, 16)))
			return false;
		/* per-filter constants are requested as 16-byte runs */
		if (!aligned_to(epi.bias, 16) || !columns_aligned(epi))
			return false;
		/* two LDS layouts: the usual one (two workgroups per compute unit) and, for filters other than 3 x 3, one with a halo
		 * large enough for 256-pixel tiles under a 5 x 5 filter (one workgroup per compute unit).  Estimated cost: rounds of
		 * resident workgroups times (k-steps at the measured pace of a workgroup that shares its compute unit, 0.68 us, or has
		 * it to itself, 0.47 us, plus 3.6 us of prologue and epilogue). */
		const int64_t filter_blocks = (static_cast<int64_t>(s.K) + TILE_N - 1) / TILE_N;
		const int64_t resident = static_cast<int64_t>(persistent_workgroups(1ll << 40));
		const int steps = s.R * s.S * ((s.C * static_cast<int>(sizeof(TE)) + STEP_BYTES - 1) / STEP_BYTES);
		auto plan = [&](TileChoice &pick, bool &big)
		{
			const bool general = s.R != 3 || s.S != 3; /* the instance with the general k loop: either row order, either LDS layout */
			pick = choose_tile(s, HALO_SMALL, TileLds<HALO_SMALL>::pixels, general);
			big = false;
			if (general)
			{
				const TileChoice wide = choose_tile(s, HALO_BIG, TileLds<HALO_BIG>::pixels, true);
				if (wide.tiles > 0)
				{
					const int64_t wide_groups = static_cast<int64_t>(s.N) * wide.tiles * filter_blocks, groups = static_cast<int64_t>(s.N) * pick.tiles * filter_blocks;
					const double wide_cost = static_cast<double>((wide_groups + resident / 2 - 1) / (resident / 2)) * (steps * 0.47 + 3.6);
					const double cost = static_cast<double>((groups + resident - 1) / resident) * (steps * (groups > resident / 2 ? 0.68 : 0.47) + 3.6);
					/* (tiles that would be mostly padding send the layer to the gather kernel, see below: then the other layout is
					 * the only candidate) */
					const bool mostly_padding = pick.tiles > 0 && static_cast<double>(s.Ho) * s.Wo < 0.5 * pick.tiles * TILE_M;
					if (pick.tiles == 0 || mostly_padding || wide_cost < 0.9 * cost)
					{
						pick = wide;
						big = true;
					}
				}
			}
		};
		/* the search walks a few thousand candidate tiles: a caller that issues the same layer again (a network does nothing
		 * else) gets the answer of the last search of its thread */
		struct Plan
		{
			int N, Ho, Wo, R, S, K, C, element;
			TileChoice pick;
			bool big;
		};
		static thread_local Plan last = { 0, 0, 0, 0, 0, 0, 0, 0, { 0, 0, 0, 0 }, false };
		TileChoice pick;
		bool big;
		if (last.N == s.N && last.Ho == s.Ho && last.Wo == s.Wo && last.R == s.R && last.S == s.S && last.K == s.K && last.C == s.C
				&& last.element == static_cast<int>(sizeof(TE)))
		{
			pick = last.pick;
			big = last.big;
		}
		else
		{
			plan(pick, big);
			last = { s.N, s.Ho, s.Wo, s.R, s.S, s.K, s.C, static_cast<int>(sizeof(TE)), pick, big };
		}
		if (pick.tiles == 0)
			return false;
		TileGeom g;
		g.TH = pick.th;
		g.TW = pick.tw;
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
		g.flip = s.mode != 0 ? 1 : 0;
		g.HH = g.TH + s.R - 1;
		g.HW = g.TW + s.S - 1;
		g.hw_magic = (1u << 20) / static_cast<unsigned int>(g.HW) + 1u; /* HW <= 448 and the dividends are below 512 */
		g.row_pitch = pick.dense ? g.TW : g.HW;
		g.row_magic = (1u << 20) / static_cast<unsigned int>(g.row_pitch) + 1u; /* dividends below 256 */
		g.tiles_h = (s.Ho + g.TH - 1) / g.TH;
		g.tiles_w = (s.Wo + g.TW - 1) / g.TW;
		g.slices = (s.C * static_cast<int>(sizeof(TE)) + STEP_BYTES - 1) / STEP_BYTES;
		g.images = s.N;
		/* the gather kernel wastes nothing on partially filled tiles: keep it when tiles would be mostly padding */
		const double fill = static_cast<double>(s.Ho) * s.Wo / (static_cast<double>(g.tiles_h) * g.tiles_w * TILE_M);
		if (fill < 0.5)
			return false;
		if (static_cast<int64_t>(s.Ho) * s.Wo * s.K >= (1ll << 31))
			return false;
		/* 24-bit multiplications in the halo addressing */
		if (static_cast<int64_t>(s.W) * s.C * static_cast<int64_t>(sizeof(TE)) >= (1 << 24))
			return false;
		const int64_t blocks = static_cast<int64_t>(s.N) * g.tiles_h * g.tiles_w;
		if (blocks * filter_blocks > 0x7FFFFFFFll)
			return false;
		g.filter_blocks = static_cast<int>(filter_blocks);
		g.filter_shift = -1;
		for (int sh = 0; sh < 31; sh++)
			if ((1ll << sh) == filter_blocks)
				g.filter_shift = sh;
		g.filter_fastest = blocks * filter_blocks > static_cast<int64_t>(persistent_workgroups(1ll << 40)) ? 1 : 0;
		const dim3 grid(static_cast<unsigned int>(blocks * filter_blocks));
		if (s.R == 3 && s.S == 3)
			hipLaunchKernelGGL((k_conv_tile<TE, Epi, 3>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		else if (big && s.R == 5 && s.S == 5 && g.slices == 1)
			hipLaunchKernelGGL((k_conv_tile<TE, Epi, 5, HALO_BIG>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		else if (big)
			hipLaunchKernelGGL((k_conv_tile<TE, Epi, 0, HALO_BIG>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		else
			hipLaunchKernelGGL((k_conv_tile<TE, Epi, 0>), grid, dim3(256), 0, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi);
		return true;
	}

#define AVHIP_INSTANTIATE(TE, EPI) template bool conv_tile_launch<TE, EPI>(hipStream_t, const avhipConvShape&, const void*, const void*, const EPI&);
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
