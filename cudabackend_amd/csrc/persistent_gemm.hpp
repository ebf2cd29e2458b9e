/*
 * persistent_gemm.hpp -- a batched NT product  C[b][rows, cols] = A[b][rows, k] * B[b][cols, k]^T  with a SHORT k, run by
 * workgroups that stay on their compute unit and walk a sequence of 128 x 128 (or 64 x 128) tiles as one software pipeline.
 *
 * Used where k is so short (at most four 128-byte steps) that a workgroup computing a single tile spends most of its life
 * waiting for its first operands and draining its accumulators: 1x1 convolutions (conv_pointwise.hip) and the batched GEMM
 * of non-fused Winograd (gemm.hip), whose k is the channel count.  Same MFMA shapes, LDS layout and drain as the one-tile
 * engine of mfma_core.hpp; the schedule differs:
 *   - A: every k-step of a tile has its own register set, and a set is refilled with the same step of the NEXT tile right
 *     after it went to LDS, so the A rows of a tile are requested before the previous tile is drained;
 *   - B: fetched two k-steps ahead, across tile boundaries (a register set per step for B as well spills and was measured
 *     slower);
 *   - the accumulators of a finished tile leave through the LDS buffer that tile no longer needs while the other buffer
 *     already holds the first step of the next tile;
 *   - per-column constants of the epilogue (bias, scale) are staged in LDS for all columns once: a global load per tile
 *     would make every tile wait for the whole memory counter.
 * Tiles are numbered (batch, row block, column block) with the column block fastest and each XCD takes a contiguous run of
 * them, so the workgroups that share a block of A rows run at the same time behind the same L2 and A comes from HBM once.
 *
 * The epilogue type provides: scalar_t, wide, ColumnsT<W>, pin(), load_columns(col, ColumnsT<1>&),
 * pick_columns(table, col, ColumnsT<W>&), store_at<ACT_SIMPLE, true, W>(element index, col, values, columns) and, when its
 * masked_stores is set, store_masked<W>(exists, element index, col, values, columns, sink) with out_bytes and out().
 */
#ifndef AVHIP_PERSISTENT_GEMM_HPP_
#define AVHIP_PERSISTENT_GEMM_HPP_

#include <atomic>

#include "conv_epilogue.hpp"
#include "mfma_core.hpp"

namespace avhip
{
	constexpr int PERSISTENT_TABLE_BYTES = 8192; /* LDS left for the per-column constants with two workgroups per compute unit */
	constexpr int PERSISTENT_LDS_BYTES = LDS_BYTES + PERSISTENT_TABLE_BYTES;
	constexpr int PERSISTENT_MAX_STEPS = 4;

	struct PersistentGeom
	{
		int rows, cols; /* of one batch member */
		unsigned int row_bytes; /* k * sizeof(TE) */
		unsigned int a_pitch, b_pitch; /* bytes between consecutive rows of A and of B */
		unsigned int a_batch, b_batch; /* bytes between consecutive batch members */
		unsigned int a_bytes, b_bytes; /* extent of all of A and of B (below 2 GiB) */
		int64_t c_batch; /* elements between batch members of C */
		int c_pitch; /* elements between rows of C (below 2^22: the byte offset of a tile's last row is a 32-bit product) */
		int row_blocks, col_blocks; /* ceil(rows / tile rows), ceil(cols / 128) */
		int tiles; /* batch * row_blocks * col_blocks */
		int table_columns; /* columns whose constants are staged in LDS (cols, or 0 when the epilogue has none) */
	};

	/* Splits a tile number into (batch member, row block, column block). */
	struct PersistentTile
	{
		int batch, row_block, col_block;
	};
	__device__ inline PersistentTile persistent_tile(const PersistentGeom &g, int tile)
	{
		const unsigned int t = static_cast<unsigned int>(tile);
		const unsigned int rc = t / static_cast<unsigned int>(g.col_blocks);
		PersistentTile r;
		r.col_block = static_cast<int>(t - rc * g.col_blocks);
		r.batch = static_cast<int>(rc / static_cast<unsigned int>(g.row_blocks));
		r.row_block = static_cast<int>(rc - static_cast<unsigned int>(r.batch) * g.row_blocks);
		return r;
	}

	/* STEPS: k-steps per tile, even (an odd count is rounded up and the extra step reads zeros).  TM: the tile has 64 * TM rows
	 * (each of the 2 x 2 wavefronts takes TM 32-row MFMA tiles by two 32-column ones); g.row_blocks counts blocks of that
	 * height.  TM = 1 halves the tile for products so slow per tile (fp32) that evening out the rounds matters more than
	 * operand reuse.  Called by all 256 work-items of a workgroup with PERSISTENT_LDS_BYTES of LDS; gridDim.x workgroups share
	 * the tiles. */
	template<typename TE, typename Epi, int STEPS, int TM = 2>
	__device__ __forceinline__ void persistent_nt_gemm(char *lds, const TE *__restrict__ A, const TE *__restrict__ B, const PersistentGeom &g, Epi &epi)
	{
		static_assert(STEPS % 2 == 0 && STEPS <= PERSISTENT_MAX_STEPS, "register sets and LDS buffers alternate with the step parity");
		static_assert(TM == 1 || TM == 2, "64 or 128 rows");
		constexpr int ROWS = 64 * TM;
		constexpr int A_PASSES = ROWS / FETCH_ROWS;
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
		const int rd_a = (wm * 32 * TM + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;
		const int rd_b = (wn * 64 + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;
		const __amdgpu_buffer_rsrc_t ra_rsrc = make_buffer(A, g.a_bytes);
		const __amdgpu_buffer_rsrc_t rb_rsrc = make_buffer(B, g.b_bytes);

		/* tile sequence of this workgroup: in round j it takes tile j * gridDim.x + (its number within the round).  In full
		 * rounds that number is XCD-contiguous (neighbouring tiles share rows of A behind one L2); the last, partial round hands
		 * its tiles out by plain workgroup number, which spreads them over all XCDs instead of filling the first ones. */
		const int in_full_round = xcd_block(blockIdx.x, gridDim.x);
		const int full_rounds = g.tiles / static_cast<int>(gridDim.x);
		auto tile_of = [&](int round) { return round * static_cast<int>(gridDim.x) + (round < full_rounds ? in_full_round : static_cast<int>(blockIdx.x)); };

		/* the two fetch cursors: A one tile ahead of the MFMAs, B two steps ahead */
		int a_round = 0, a_step = 0, b_round = 0, b_step = 0;
		unsigned int a_base[A_PASSES], b_base[FETCH_PASSES];
		auto aim_a = [&]()
		{
			const int a_tile = tile_of(a_round);
			const bool live = a_tile < g.tiles;
			const PersistentTile t = persistent_tile(g, live ? a_tile : 0);
#pragma unroll
			for (int q = 0; q < A_PASSES; q++)
			{
				const int r = t.row_block * ROWS + frow + FETCH_ROWS * q;
				a_base[q] = (live && r < g.rows) ? static_cast<unsigned int>(t.batch) * g.a_batch + static_cast<unsigned int>(r) * g.a_pitch + fpart * 16 :
						OUT_OF_RANGE;
			}
		};
		auto aim_b = [&]()
		{
			const int b_tile = tile_of(b_round);
			const bool live = b_tile < g.tiles;
			const PersistentTile t = persistent_tile(g, live ? b_tile : 0);
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int c = t.col_block * BLOCK_N + frow + FETCH_ROWS * q;
				b_base[q] = (live && c < g.cols) ? static_cast<unsigned int>(t.batch) * g.b_batch + static_cast<unsigned int>(c) * g.b_pitch + fpart * 16 :
						OUT_OF_RANGE;
			}
		};
		auto fetch_a = [&](uint4 (&a)[A_PASSES]) __attribute__((always_inline))
		{
			const unsigned int k_byte = static_cast<unsigned int>(a_step) * STEP_BYTES;
			const bool in_row = k_byte + fpart * 16 < g.row_bytes;
#pragma unroll
			for (int q = 0; q < A_PASSES; q++)
				a[q] = buffer_fetch(ra_rsrc, (in_row && a_base[q] < OUT_OF_RANGE) ? a_base[q] + k_byte : OUT_OF_RANGE);
			if (++a_step == STEPS)
			{
				a_step = 0;
				a_round++;
				aim_a();
			}
		};
		auto fetch_b = [&](uint4 (&b)[FETCH_PASSES]) __attribute__((always_inline))
		{
			const unsigned int k_byte = static_cast<unsigned int>(b_step) * STEP_BYTES;
			const bool in_row = k_byte + fpart * 16 < g.row_bytes;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
				b[q] = buffer_fetch(rb_rsrc, (in_row && b_base[q] < OUT_OF_RANGE) ? b_base[q] + k_byte : OUT_OF_RANGE);
			if (++b_step == STEPS)
			{
				b_step = 0;
				b_round++;
				aim_b();
			}
		};
		auto stash = [&](int buffer, const uint4 (&a)[A_PASSES], const uint4 (&b)[FETCH_PASSES]) __attribute__((always_inline))
		{
			char *sa = lds + buffer * 2 * LDS_TILE;
			char *sb = sa + LDS_TILE;
#pragma unroll
			for (int q = 0; q < A_PASSES; q++)
				*reinterpret_cast<uint4*>(sa + st_off + q * FETCH_ROWS * LDS_ROW) = a[q];
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
				*reinterpret_cast<uint4*>(sb + st_off + q * FETCH_ROWS * LDS_ROW) = b[q];
		};

		typename Mma<TE>::acc_t acc[TM][2];
		auto multiply = [&](int buffer) __attribute__((always_inline))
		{
			const char *sa = lds + buffer * 2 * LDS_TILE;
			const char *sb = sa + LDS_TILE;
			constexpr int SLABS = STEP_BYTES / 32;
			Chunk a[2][TM], b[2][2]; /* LDS reads run one 32-byte slab ahead of the MFMAs */
			auto read = [&](int slab, Chunk (&ra_)[TM], Chunk (&rb_)[2]) __attribute__((always_inline))
			{
#pragma unroll
				for (int i = 0; i < TM; i++)
					ra_[i].u = *reinterpret_cast<const uint4*>(sa + rd_a + i * 32 * LDS_ROW + slab * 32);
#pragma unroll
				for (int i = 0; i < 2; i++)
					rb_[i].u = *reinterpret_cast<const uint4*>(sb + rd_b + i * 32 * LDS_ROW + slab * 32);
			};
			read(0, a[0], b[0]);
#pragma unroll
			for (int slab = 0; slab < SLABS; slab++)
			{
				if (slab + 1 < SLABS)
					read(slab + 1, a[(slab + 1) & 1], b[(slab + 1) & 1]);
				if (sizeof(TE) < 4)
					burst_priority(slab);
#pragma unroll
				for (int i = 0; i < TM; i++)
#pragma unroll
					for (int j = 0; j < 2; j++)
						Mma<TE>::run(a[slab & 1][i], b[slab & 1][j], acc[i][j]);
				if (sizeof(TE) < 4 && slab + 1 == SLABS)
					__builtin_amdgcn_s_setprio(0);
			}
		};

		/* prologue: all of the first tile's A, two steps of B, step 0 into LDS, and set 0 of A goes on to the second tile */
		uint4 ra[STEPS][A_PASSES], rb[2][FETCH_PASSES];
		aim_a();
		aim_b();
#pragma unroll
		for (int s = 0; s < STEPS; s++)
			fetch_a(ra[s]);
		fetch_b(rb[0]);
		fetch_b(rb[1]);
		for (int c = tid; c < g.table_columns; c += 256)
			epi.load_columns(c, table[c]);
		stash(0, ra[0], rb[0]);
		fetch_a(ra[0]);
		if constexpr (Epi::masked_stores)
		{
			/* The compiler counts the vector-memory operations in flight statically and, where two paths meet, assumes the
			 * shorter queue.  The first tile is entered from here, every later one from behind the stores of the drain: as
			 * many stores that go nowhere (empty buffer: dropped by the hardware) make the two queues equal, so the waits of
			 * the tile loop allow the drain's stores to be in flight instead of waiting for them. */
			const __amdgpu_buffer_rsrc_t nowhere = make_buffer(epi.out(), 0);
			typedef unsigned int drain_words_t __attribute__((ext_vector_type(W * Epi::out_bytes / 4)));
			const drain_words_t nothing = {};
#pragma unroll
			for (int i = 0; i < DrainRows<TM, 2, W>::slots; i++)
				buffer_put(nowhere, OUT_OF_RANGE + 16u * i, nothing); /* distinct offsets, or the compiler keeps only the last */
		}

		const int col_in_tile = drain_column<2, W>();
		for (int round = 0; tile_of(round) < g.tiles; round++)
		{
			const PersistentTile t = persistent_tile(g, tile_of(round));
			const int col = t.col_block * BLOCK_N + col_in_tile;
#pragma unroll
			for (int i = 0; i < TM; i++)
#pragma unroll
				for (int j = 0; j < 2; j++)
#pragma unroll
					for (int v = 0; v < 16; v++)
						acc[i][j][v] = 0;
			/* step s is multiplied from LDS buffer s % 2; meanwhile step s + 2 of B is requested into the set step s just
			 * left, step s + 1 goes to the other buffer, and the A set it came from is refilled for the next tile */
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
			const int64_t c_tile = static_cast<int64_t>(t.batch) * g.c_batch + static_cast<int64_t>(t.row_block * ROWS) * g.c_pitch + t.col_block * BLOCK_N;
			const int64_t c0 = c_tile + col_in_tile; /* element index of (first row of the tile, this work-item's first column) */
			const int row0 = t.row_block * ROWS;
			typename Epi::template ColumnsT<W> columns;
			if (col < g.table_columns)
				Epi::pick_columns(table, col, columns);
			if constexpr (Epi::masked_stores)
			{
				/* every work-item issues every store, rows and columns that do not exist at an out-of-range offset: a store
				 * behind a condition would make each later wait for the next tile's operands wait for the stores as well */
				const __amdgpu_buffer_rsrc_t rc = make_buffer(epi.out() + c_tile * Epi::out_bytes, 0x7FFFFFF0u);
				auto run_offset = [&](int r) __attribute__((always_inline))
				{
					return (row0 + r < g.rows && col < g.cols) ? static_cast<unsigned int>(r * g.c_pitch + col_in_tile) * Epi::out_bytes : OUT_OF_RANGE;
				};
				if constexpr (Epi::residual_ahead)
				{
					/* the residual of the rows of a pass is requested before the pass goes through LDS, unconditionally (no
					 * residual: an empty buffer), instead of row by row between the stores */
					typedef DrainRows<TM, 2, W> Rows;
					const bool has_z = epi.residual() != nullptr;
					const __amdgpu_buffer_rsrc_t rz = make_buffer(has_z ? epi.residual() + c_tile * Epi::out_bytes : nullptr, has_z ? 0x7FFFFFF0u : 0u);
					typename Epi::template Residual<W> residual[Rows::iterations];
					drain_tile<TE, TM, 2, W>(lds + 2 * LDS_TILE, acc, [&](int r, const typename Epi::scalar_t (&v)[W], int slot) __attribute__((always_inline))
					{
						const unsigned int offset = run_offset(r);
						epi.template store_masked<W>(offset != OUT_OF_RANGE, c0 + r * g.c_pitch, col, v, columns, [&](auto words) __attribute__((always_inline))
						{
							buffer_put<STORE_STREAM_THROUGH>(rc, offset, words);
						}, &residual[slot % Rows::iterations]);
					}, [&](int tm) __attribute__((always_inline))
					{
#pragma unroll
						for (int it = 0; it < Rows::iterations; it++)
						{
							union
							{
								uint4 u;
								decltype(residual[0].raw) p;
							} cast;
							cast.u = buffer_fetch(rz, run_offset(Rows::row(tm * Rows::iterations + it)));
							residual[it].raw = cast.p;
						}
					});
				}
				else
					drain_tile<TE, TM, 2, W>(lds + 2 * LDS_TILE, acc, [&](int r, const typename Epi::scalar_t (&v)[W], int) __attribute__((always_inline))
					{
						const unsigned int offset = run_offset(r);
						epi.template store_masked<W>(offset != OUT_OF_RANGE, c0 + r * g.c_pitch, col, v, columns, [&](auto words) __attribute__((always_inline))
						{
							buffer_put<STORE_STREAM_THROUGH>(rc, offset, words);
						});
					});
			}
			else
				drain_tile<TE, TM, 2, W>(lds + 2 * LDS_TILE, acc, [&](int r, const typename Epi::scalar_t (&v)[W], int) __attribute__((always_inline))
				{
					if (row0 + r < g.rows && col < g.cols)
						epi.template store_at<ACT_SIMPLE, true, W>(c0 + r * g.c_pitch, col, v, columns);
				});
		}
	}

	/* Which engine runs short-k NT products (1x1 convolutions, the batched GEMM of non-fused Winograd): 0 = B resident in
	 * registers (resident_gemm.hpp, the default), 1 = both operands through LDS (this file).  Set by avhip_set_short_k_engine. */
	std::atomic<int>& short_k_engine();

	/* How many workgroups to launch: two per compute unit stay resident; with fewer tiles every workgroup has one. */
	inline unsigned int persistent_workgroups(int64_t tiles)
	{
		static std::atomic<int> known_units[64]; /* per device, 0 = not asked yet; the answer never changes */
		int device = 0, units = 0;
		if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64)
			device = -1;
		if (device >= 0)
			units = known_units[device].load(std::memory_order_relaxed);
		if (units <= 0)
		{
			if (device < 0 || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0)
				units = 256;
			else
				known_units[device].store(units, std::memory_order_relaxed);
		}
		const int64_t resident = 2 * static_cast<int64_t>(units);
		return static_cast<unsigned int>(tiles < resident ? tiles : resident);
	}
}

#endif /* AVHIP_PERSISTENT_GEMM_HPP_ */
