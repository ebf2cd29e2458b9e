/*
 * resident_gemm.hpp -- a batched NT product  C[b][rows, cols] = A[b][rows, k] * B[b][cols, k]^T  with a SHORT k (at most four
 * 128-byte steps) in which the B operand never touches LDS: every wavefront keeps the B rows of its 32 output columns, all of
 * k, in registers for as long as it works on that column block, and only A streams.
 *
 * Why: a compute unit takes in 64 bytes per clock from L2.  A 128 x 128 tile that loads 128 rows of A and 128 rows of B per
 * k-step needs 512 clocks of that path for 512 clocks of MFMAs, so the one-tile-per-step engines (mfma_core.hpp,
 * persistent_gemm.hpp) are bound by operand traffic, not by the matrix cores.  With B resident the same MFMAs need half the
 * traffic, half the LDS writes and no LDS reads for B.  It fits because k is short: 32 columns x 512 bytes are 64 registers.
 *
 * Work split: a unit is (batch member, column block of 128, a contiguous range of rows); the rows of a (batch member, column
 * block) are cut into `splits` ranges of whole 32-row granules, as even as possible.  Units are numbered with the column block
 * fastest and handed out XCD-contiguously, so the workgroups that read the same rows of A run at the same time behind the
 * same L2.  A workgroup (4 wavefronts, each 32 * TM rows x 32 columns = TM 32 x 32 MFMA tiles) walks its range in tiles of
 * 32 * TM rows; a last tile that is at most half full runs an instance that multiplies half the granules (a run-time granule
 * count inside one instance costs registers: measured, it spills).  TM = 2 measured faster than TM = 4 on every shape tried
 * (64-row tiles even out the ranges and leave registers for the epilogue); two workgroups per compute unit.
 *
 * Pipeline per k-step q (flattened over the tiles of a unit; register sets R0 / R1 and LDS buffers L0 / L1 alternate):
 *     barrier;  R[q % 2] <- global A of step q + 2;  MFMAs of step q from L[q % 2] and the B registers;  L[(q+1) % 2] <- R[(q+1) % 2]
 * The accumulators of a finished tile leave through a private LDS area of each wavefront (no workgroup barrier), 16 bytes
 * per work-item and store.
 *
 * The epilogue type provides what persistent_gemm.hpp asks of it.
 */
#ifndef AVHIP_RESIDENT_GEMM_HPP_
#define AVHIP_RESIDENT_GEMM_HPP_

#include <type_traits>

#include "conv_epilogue.hpp"
#include "mfma_core.hpp"
#include "persistent_gemm.hpp"

namespace avhip
{
	constexpr int RESIDENT_DRAIN_PITCH = 40; /* words per row of a wavefront's 32 x 32 hand-over area: rows 16-byte aligned, the two half-wavefronts on disjoint banks */
	constexpr int RESIDENT_DRAIN_BYTES = 32 * RESIDENT_DRAIN_PITCH * 4; /* per wavefront */
	constexpr int RESIDENT_TABLE_BYTES = 8192;
	constexpr int RESIDENT_TM = 2; /* 32-row granules per tile */
	constexpr int RESIDENT_OCCUPANCY = 2; /* workgroups per compute unit the kernels are built for */
	template<int TM> struct ResidentLds
	{
		static constexpr int tile = 32 * TM * LDS_ROW; /* one k-step of the A rows of a tile */
		static constexpr int bytes = 2 * tile + 4 * RESIDENT_DRAIN_BYTES + RESIDENT_TABLE_BYTES;
	};
	constexpr int RESIDENT_LDS_BYTES = ResidentLds<RESIDENT_TM>::bytes;
	constexpr int RESIDENT_MAX_STEPS = 4;
	constexpr int RESIDENT_COLS = 128, RESIDENT_GRANULE = 32;

	struct ResidentGeom
	{
		int rows, cols; /* of one batch member */
		unsigned int row_bytes; /* k * sizeof(TE), a multiple of 16 */
		unsigned int a_pitch, b_pitch; /* bytes between consecutive rows of A and of B */
		unsigned int a_batch, b_batch; /* bytes between consecutive batch members */
		unsigned int a_bytes, b_bytes; /* extent of all of A and of B (below 2 GiB) */
		int64_t c_batch; /* elements between batch members of C */
		int c_pitch; /* elements between rows of C (below 2^22) */
		int col_blocks; /* ceil(cols / 128) */
		int splits; /* row ranges per (batch member, column block) */
		int granules; /* ceil(rows / 32) */
		int units; /* batch * splits * col_blocks */
		int table_columns; /* columns whose epilogue constants are staged in LDS (cols, or 0 when the epilogue has none) */
	};

	/* Fills splits / granules / units for `batch` members and returns the number of workgroups to launch. */
	inline unsigned int resident_plan(ResidentGeom &g, int batch)
	{
		const int64_t resident = persistent_workgroups(1ll << 40) / 2 * RESIDENT_OCCUPANCY; /* workgroups that stay on the chip together */
		g.col_blocks = (g.cols + RESIDENT_COLS - 1) / RESIDENT_COLS;
		g.granules = (g.rows + RESIDENT_GRANULE - 1) / RESIDENT_GRANULE;
		const int64_t groups = static_cast<int64_t>(batch) * g.col_blocks;
		int64_t splits = resident / groups;
		const int64_t most = (g.granules + RESIDENT_TM - 1) / RESIDENT_TM; /* no range shorter than one tile while others have several */
		splits = splits < 1 ? 1 : (splits > most ? most : splits);
		g.splits = static_cast<int>(splits);
		const int64_t units = groups * splits;
		g.units = static_cast<int>(units);
		return static_cast<unsigned int>(units < resident ? units : resident);
	}

	template<typename TE, typename Epi, int STEPS, int TM = RESIDENT_TM>
	__device__ __forceinline__ void resident_nt_gemm(char *lds, const TE *__restrict__ A, const TE *__restrict__ B, const ResidentGeom &g, Epi &epi)
	{
		static_assert(STEPS >= 1 && STEPS <= RESIDENT_MAX_STEPS, "B of all k-steps lives in registers");
		constexpr int W = Epi::wide;
		constexpr int SLABS = STEP_BYTES / 32;
		constexpr int RESIDENT_ROWS = 32 * TM;
		constexpr int A_PASSES = RESIDENT_ROWS / FETCH_ROWS;
		constexpr int LDS_TILE = ResidentLds<TM>::tile; /* (shadows the 128-row constant of the shared engine) */
		typedef typename Epi::scalar_t S;
		typedef typename Epi::template ColumnsT<1> Record;
		/* hand-over of a 32 x 32 accumulator tile: TPR work-items share a row, each takes W consecutive columns */
		constexpr int TPR = 32 / W;
		constexpr int SWEEP_ROWS = 64 / TPR;
		constexpr int SWEEPS = 32 / SWEEP_ROWS;
		static_assert(W == 4 || W == 8 || W == 16, "a work-item takes 4, 8 or 16 consecutive columns");
		char *abuf = lds;
		Record *table = reinterpret_cast<Record*>(lds + 2 * LDS_TILE + 4 * RESIDENT_DRAIN_BYTES);
		epi.pin();
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		S *sm = reinterpret_cast<S*>(lds + 2 * LDS_TILE + wave * RESIDENT_DRAIN_BYTES);
		const int fpart = tid & (STEP_CHUNKS - 1);
		const int frow = tid / STEP_CHUNKS;
		const int st_off = frow * LDS_ROW + fpart * 16;
		const int rd_a = (lane & 31) * LDS_ROW + (lane >> 5) * 16;
		const __amdgpu_buffer_rsrc_t ra_rsrc = make_buffer(A, g.a_bytes);
		const __amdgpu_buffer_rsrc_t rb_rsrc = make_buffer(B, g.b_bytes);
		const int col_in_block = wave * 32 + (lane % TPR) * W; /* first of this work-item's W output columns */
		const int drain_row = lane / TPR; /* its row within a sweep */

		for (int c = tid; c < g.table_columns; c += 256)
			epi.load_columns(c, table[c]);

		for (int unit = static_cast<int>(xcd_block(blockIdx.x, gridDim.x)); unit < g.units; unit += static_cast<int>(gridDim.x))
		{
			const unsigned int u = static_cast<unsigned int>(unit);
			const unsigned int rest = u / static_cast<unsigned int>(g.col_blocks);
			const int col_block = static_cast<int>(u - rest * g.col_blocks);
			const int batch = static_cast<int>(rest / static_cast<unsigned int>(g.splits));
			const int split = static_cast<int>(rest - static_cast<unsigned int>(batch) * g.splits);
			const int row_begin = static_cast<int>(static_cast<int64_t>(split) * g.granules / g.splits) * RESIDENT_GRANULE;
			int row_end = static_cast<int>(static_cast<int64_t>(split + 1) * g.granules / g.splits) * RESIDENT_GRANULE;
			row_end = row_end < g.rows ? row_end : g.rows;

			/* B: lane l holds, for output column 32 * wave + l % 32, the 16-byte chunks (2 * slab + l / 32) of every step */
			Chunk breg[STEPS][SLABS];
			{
				const int bcol = col_block * RESIDENT_COLS + wave * 32 + (lane & 31);
				const unsigned int b_base = static_cast<unsigned int>(batch) * g.b_batch + static_cast<unsigned int>(bcol) * g.b_pitch + (lane >> 5) * 16;
#pragma unroll
				for (int s = 0; s < STEPS; s++)
#pragma unroll
					for (int j = 0; j < SLABS; j++)
					{
						const unsigned int k_byte = s * STEP_BYTES + j * 32 + (lane >> 5) * 16;
						breg[s][j].u = buffer_fetch(rb_rsrc, (bcol < g.cols && k_byte < g.row_bytes) ? b_base + s * STEP_BYTES + j * 32 : OUT_OF_RANGE);
					}
			}

			/* the A cursor runs two steps ahead of the MFMAs; rows at or past row_end read zeros */
			int f_row = row_begin, f_step = 0;
			unsigned int a_base[A_PASSES];
			auto aim = [&]() __attribute__((always_inline))
			{
#pragma unroll
				for (int q = 0; q < A_PASSES; q++)
				{
					const int r = f_row + frow + FETCH_ROWS * q;
					a_base[q] = r < row_end ? static_cast<unsigned int>(batch) * g.a_batch + static_cast<unsigned int>(r) * g.a_pitch + fpart * 16 : OUT_OF_RANGE;
				}
			};
			auto fetch = [&](uint4 (&a)[A_PASSES]) __attribute__((always_inline))
			{
				const unsigned int k_byte = static_cast<unsigned int>(f_step) * STEP_BYTES;
				const bool in_row = k_byte + fpart * 16 < g.row_bytes;
#pragma unroll
				for (int q = 0; q < A_PASSES; q++)
					a[q] = buffer_fetch(ra_rsrc, (in_row && a_base[q] != OUT_OF_RANGE) ? a_base[q] + k_byte : OUT_OF_RANGE);
				if (++f_step == STEPS)
				{
					f_step = 0;
					f_row += RESIDENT_ROWS;
					aim();
				}
			};
			auto stash = [&](int buffer, const uint4 (&a)[A_PASSES]) __attribute__((always_inline))
			{
#pragma unroll
				for (int q = 0; q < A_PASSES; q++)
					*reinterpret_cast<uint4*>(abuf + buffer * LDS_TILE + st_off + q * FETCH_ROWS * LDS_ROW) = a[q];
			};

			typename Mma<TE>::acc_t acc[TM];
			auto multiply = [&](int step, int buffer, auto granules) __attribute__((always_inline))
			{
				constexpr int GR = decltype(granules)::value; /* 32-row granules of this tile that exist */
				const char *sa = abuf + buffer * LDS_TILE + rd_a;
				Chunk a[2][TM]; /* LDS reads run one 32-byte slab ahead of the MFMAs */
				auto read = [&](int slab, Chunk (&r)[TM]) __attribute__((always_inline))
				{
#pragma unroll
					for (int tm = 0; tm < TM; tm++)
						if (tm < GR)
							r[tm].u = *reinterpret_cast<const uint4*>(sa + tm * 32 * LDS_ROW + slab * 32);
				};
				read(0, a[0]);
#pragma unroll
				for (int slab = 0; slab < SLABS; slab++)
				{
					if (slab + 1 < SLABS)
						read(slab + 1, a[(slab + 1) & 1]);
					if (sizeof(TE) < 4)
						burst_priority(slab);
#pragma unroll
					for (int tm = 0; tm < TM; tm++)
						if (tm < GR)
							Mma<TE>::run(a[slab & 1][tm], breg[step][slab], acc[tm]);
					if (sizeof(TE) < 4 && slab + 1 == SLABS)
						__builtin_amdgcn_s_setprio(0);
				}
			};

			uint4 ra[2][A_PASSES];
			aim();
			fetch(ra[0]);
			fetch(ra[1]);
			__syncthreads(); /* the table is complete; nobody still reads buffer 0 for the unit before */
			stash(0, ra[0]);
			typename Epi::template ColumnsT<W> columns;
			const int col = col_block * RESIDENT_COLS + col_in_block;
			if (col < g.table_columns)
				Epi::pick_columns(table, col, columns);

			/* one tile = STEPS steps starting on LDS buffer / register set P0, with GR of its four 32-row granules present */
			auto tile_of = [&](int row0, auto parity, auto granules) __attribute__((always_inline))
			{
				constexpr int P0 = decltype(parity)::value;
				constexpr int GR = decltype(granules)::value;
#pragma unroll
				for (int tm = 0; tm < TM; tm++)
#pragma unroll
					for (int v = 0; v < 16; v++)
						acc[tm][v] = 0;
#pragma unroll
				for (int s = 0; s < STEPS; s++)
				{
					const int b = (P0 + s) & 1;
					__syncthreads(); /* step q is visible in buffer b; everyone is done with step q - 1 in the other */
					if (b == 0)
						fetch(ra[0]);
					else
						fetch(ra[1]);
					multiply(s, b, granules);
					if (b == 0)
						stash(1, ra[1]);
					else
						stash(0, ra[0]);
				}
				/* hand-over and stores, 32 rows at a time, through this wavefront's own LDS area */
				const int64_t c_tile = static_cast<int64_t>(batch) * g.c_batch + static_cast<int64_t>(row0) * g.c_pitch + col_block * RESIDENT_COLS;
				const int64_t c0 = c_tile + col_in_block;
#pragma unroll
				for (int tm = 0; tm < TM; tm++)
				{
					if (tm >= GR)
						continue;
					typename Epi::template Residual<W> residual[SWEEPS];
					if constexpr (Epi::masked_stores)
					{
						if constexpr (Epi::residual_ahead)
						{
							/* the residual of the pass's rows is requested before the pass goes through LDS, unconditionally (no
							 * residual: an empty buffer) */
							const bool has_z = epi.residual() != nullptr;
							const __amdgpu_buffer_rsrc_t rz = make_buffer(has_z ? epi.residual() + c_tile * Epi::out_bytes : nullptr, has_z ? 0x7FFFFFF0u : 0u);
#pragma unroll
							for (int it = 0; it < SWEEPS; it++)
							{
								const int r = tm * 32 + drain_row + it * SWEEP_ROWS;
								union
								{
									uint4 u;
									decltype(residual[0].raw) p;
								} cast;
								cast.u = buffer_fetch(rz, (row0 + r < row_end && col < g.cols) ? static_cast<unsigned int>(r * g.c_pitch + col_in_block) * Epi::out_bytes :
										OUT_OF_RANGE);
								residual[it].raw = cast.p;
							}
						}
					}
#pragma unroll
					for (int i = 0; i < 4; i++)
#pragma unroll
						for (int j = 0; j < 4; j++)
							sm[(8 * i + 4 * (lane >> 5) + j) * RESIDENT_DRAIN_PITCH + (lane & 31)] = acc[tm][4 * i + j];
					__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront"); /* LDS serves a wavefront's accesses in order */
					typedef S quad_t __attribute__((ext_vector_type(4)));
					quad_t vals[SWEEPS][W / 4];
#pragma unroll
					for (int it = 0; it < SWEEPS; it++)
#pragma unroll
						for (int part = 0; part < W / 4; part++)
							vals[it][part] = *reinterpret_cast<const quad_t*>(sm + (drain_row + it * SWEEP_ROWS) * RESIDENT_DRAIN_PITCH + (lane % TPR) * W + 4 * part);
					__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront"); /* the next pass overwrites what was just read */
#pragma unroll
					for (int it = 0; it < SWEEPS; it++)
					{
						S v[W];
#pragma unroll
						for (int q = 0; q < W; q++)
							v[q] = vals[it][q / 4][q % 4];
						const int r = tm * 32 + drain_row + it * SWEEP_ROWS;
						const bool exists = row0 + r < row_end && col < g.cols;
						const int64_t idx = c0 + static_cast<int64_t>(r) * g.c_pitch;
						if constexpr (Epi::masked_stores)
						{
							/* every work-item issues every store, runs that do not exist at an out-of-range offset: a store behind a
							 * condition would make each later wait for A wait for the stores as well */
							const __amdgpu_buffer_rsrc_t rc = make_buffer(epi.out() + c_tile * Epi::out_bytes, 0x7FFFFFF0u);
							const unsigned int offset = exists ? static_cast<unsigned int>(r * g.c_pitch + col_in_block) * Epi::out_bytes : OUT_OF_RANGE;
							if constexpr (Epi::residual_ahead)
								epi.template store_masked<W>(exists, idx, col, v, columns, [&](auto words) __attribute__((always_inline))
								{
									buffer_put<STORE_STREAM_THROUGH>(rc, offset, words);
								}, &residual[it]);
							else
								epi.template store_masked<W>(exists, idx, col, v, columns, [&](auto words) __attribute__((always_inline))
								{
									buffer_put<STORE_STREAM_THROUGH>(rc, offset, words);
								});
						}
						else
						{
							if (exists)
								epi.template store_at<ACT_SIMPLE, true, W>(idx, col, v, columns);
						}
					}
				}
			};
			/* full tiles take the straight-line instance; the last tile of a range picks the instance for the granules it has, so
			 * that a range costs its rows rounded up to 64, not to 128 (branches inside one instance cost registers: spills) */
			auto tile = [&](int row0, auto parity) __attribute__((always_inline))
			{
				if (row_end - row0 > RESIDENT_ROWS / 2)
					tile_of(row0, parity, std::integral_constant<int, TM>());
				else
					tile_of(row0, parity, std::integral_constant<int, TM / 2>());
			};
			if constexpr (STEPS % 2 == 0)
			{
				for (int row0 = row_begin; row0 < row_end; row0 += RESIDENT_ROWS)
					tile(row0, std::integral_constant<int, 0>());
			}
			else
			{
				/* an odd step count flips the buffer parity from tile to tile: two tiles per trip keep it a compile-time constant */
				for (int row0 = row_begin; row0 < row_end; row0 += 2 * RESIDENT_ROWS)
				{
					tile(row0, std::integral_constant<int, 0>());
					if (row0 + RESIDENT_ROWS < row_end)
						tile(row0 + RESIDENT_ROWS, std::integral_constant<int, 1>());
				}
			}
		}
	}
}

#endif /* AVHIP_RESIDENT_GEMM_HPP_ */
