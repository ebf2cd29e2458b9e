/*
 * mfma_core.hpp -- the shared block-level matrix-multiply engine on gfx950 matrix cores.
 *
 * Both the batched GEMM of the non-fused Winograd path and the implicit-GEMM convolution compute
 *     D[row, col] = sum_k A[row, k] * B[col, k]
 * with both operands contiguous along k ("NT" form), so they share one engine and differ only in how a 16-byte chunk
 * of an operand row is fetched (a plain strided matrix, or an NHWC pixel / a filter tap gathered on the fly) and in
 * what the epilogue does with an accumulator.
 *
 * Geometry (one workgroup = 256 work-items = 4 wavefronts of 64):
 *   workgroup tile 128 x 128, wavefront tile 64 x 64 = 2 x 2 MFMA tiles of 32 x 32;
 *   one k-step consumes 128 bytes of every operand row (64 fp16/bf16, 128 int8, 32 fp32 values);
 *   per step each work-item moves four 16-byte chunks of A and four of B: global -> registers -> LDS; global loads run two
 *   steps ahead of the MFMAs (two register sets) and LDS is double buffered, so there is one barrier per step;
 *   LDS rows are padded from 128 to 144 bytes so that the 32 rows a wavefront reads with one ds_read_b128 spread over banks;
 *   two workgroups fit the 160 KB of LDS of a CU.
 * MFMA shapes: v_mfma_f32_32x32x16_{f16,bf16}, v_mfma_i32_32x32x32_i8, v_mfma_f32_32x32x2_f32 (four per 16-byte chunk).
 * Lane l of a wavefront supplies row (l % 32) of the operand tile and the k-chunk (l / 32); it receives, for output column
 * (l % 32), the 16 rows 8*i + 4*(l / 32) + j (i, j < 4).
 */
#ifndef AVHIP_MFMA_CORE_HPP_
#define AVHIP_MFMA_CORE_HPP_

#include "common.hpp"
#include <type_traits>

namespace avhip
{
	typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
	typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
	typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
	typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4_t;
	typedef __attribute__((__vector_size__(16 * sizeof(int)))) int i32x16_t;

	union Chunk
	{
		uint4 u;
		bf16x8_t bf;
		f16x8_t hf;
		i32x4_t i4;
		float f[4];
	};

	/* One 32 x 32 accumulator tile and the MFMA that feeds it from two 16-byte operand chunks. */
	template<typename TE> struct Mma;
	template<> struct Mma<bf16_t>
	{
		typedef f32x16_t acc_t;
		typedef float scalar_t;
		__device__ static inline void run(const Chunk &a, const Chunk &b, acc_t &c)
		{
			c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.bf, b.bf, c, 0, 0, 0);
		}
		/* the first product of an accumulator: C is the constant zero, so no register has to be cleared beforehand */
		__device__ static inline void start(const Chunk &a, const Chunk &b, acc_t &c)
		{
			const acc_t zero = {};
			c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.bf, b.bf, zero, 0, 0, 0);
		}
	};
	template<> struct Mma<f16_t>
	{
		typedef f32x16_t acc_t;
		typedef float scalar_t;
		__device__ static inline void run(const Chunk &a, const Chunk &b, acc_t &c)
		{
			c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.hf, b.hf, c, 0, 0, 0);
		}
		__device__ static inline void start(const Chunk &a, const Chunk &b, acc_t &c)
		{
			const acc_t zero = {};
			c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.hf, b.hf, zero, 0, 0, 0);
		}
	};
	template<> struct Mma<int8_t>
	{
		typedef i32x16_t acc_t;
		typedef int scalar_t;
		__device__ static inline void run(const Chunk &a, const Chunk &b, acc_t &c)
		{
			c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a.i4, b.i4, c, 0, 0, 0);
		}
		__device__ static inline void start(const Chunk &a, const Chunk &b, acc_t &c)
		{
			const acc_t zero = {};
			c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a.i4, b.i4, zero, 0, 0, 0);
		}
	};
	template<> struct Mma<float>
	{
		typedef f32x16_t acc_t;
		typedef float scalar_t;
		__device__ static inline void run(const Chunk &a, const Chunk &b, acc_t &c)
		{
#pragma unroll
			for (int i = 0; i < 4; i++)
				c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.f[i], b.f[i], c, 0, 0, 0);
		}
		__device__ static inline void start(const Chunk &a, const Chunk &b, acc_t &c)
		{
			const acc_t zero = {};
			c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.f[0], b.f[0], zero, 0, 0, 0);
#pragma unroll
			for (int i = 1; i < 4; i++)
				c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.f[i], b.f[i], c, 0, 0, 0);
		}
	};

	/* Fetches 16 bytes starting at p; only the first `valid` elements exist (valid <= 0: all zero).  `vector_ok` says
	 * that p is 16-byte aligned whenever the chunk is complete. */
	template<typename TE>
	__device__ inline uint4 fetch_chunk(const TE *p, int valid, bool vector_ok)
	{
		constexpr int E = 16 / sizeof(TE);
		if (valid >= E && vector_ok)
			return *reinterpret_cast<const uint4*>(p);
		union
		{
			uint4 u;
			TE e[E];
		} t;
		t.u = make_uint4(0u, 0u, 0u, 0u);
		if (valid > 0)
		{
#pragma unroll
			for (int i = 0; i < E; i++)
				if (i < valid)
					t.e[i] = p[i];
		}
		return t.u;
	}
	/*
	 * Fast-path operand fetch: a raw buffer load of 16 bytes at a 32-bit byte offset into a tensor.  The hardware returns
	 * zeros for offsets beyond the buffer, so "this chunk does not exist" (outside the image, past the last row, past the
	 * last channel) is expressed by the offset OUT_OF_RANGE: no branch, no select and nothing that would have to wait for
	 * the data before the next load is issued.  Tensors on this path are smaller than 2 GiB.
	 */
	typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4_t;
	constexpr unsigned int OUT_OF_RANGE = 0x80000000u;
	/* Every descriptor made here is the same for all work-items of a wavefront (a tensor, an image, a tile of a workgroup).
	 * Saying so (readfirstlane) keeps it in scalar registers even where its address or extent came out of 64-bit arithmetic
	 * that the compiler does on the vector unit; a descriptor it believes to vary per work-item costs a loop around every
	 * load and store that uses it, and the loop's block boundaries keep those accesses from being scheduled among the MFMAs. */
	__device__ inline __amdgpu_buffer_rsrc_t make_buffer(const void *base, unsigned int bytes)
	{
		const uint64_t address = reinterpret_cast<uint64_t>(base);
		const uint64_t lo = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(address & 0xFFFFFFFFu)));
		const uint64_t hi = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(address >> 32)));
		return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(hi << 32 | lo), 0, __builtin_amdgcn_readfirstlane(static_cast<int>(bytes)), 0x00020000);
	}
	template<int POLICY = 0>
	__device__ inline uint4 buffer_fetch(__amdgpu_buffer_rsrc_t rsrc, unsigned int byte_offset)
	{
		const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(byte_offset), 0, POLICY);
		return make_uint4(v[0], v[1], v[2], v[3]);
	}
	/* The store counterpart: 16 or 8 bytes at a 32-bit byte offset, non-temporal (the writing kernel never reads them back);
	 * a store at OUT_OF_RANGE is dropped by the hardware, so "this row does not exist" needs no branch around the store. */
	typedef __attribute__((__vector_size__(2 * sizeof(unsigned int)))) unsigned int u32x2_t;
	constexpr int STORE_STREAM = 2; /* nt */
#ifndef AVHIP_STREAM_THROUGH_POLICY
#define AVHIP_STREAM_THROUGH_POLICY 19
#endif
	constexpr int STORE_STREAM_THROUGH = AVHIP_STREAM_THROUGH_POLICY; /* sc0 sc1 nt: written through to memory as it goes; measured 1-3 % faster than nt alone in
	                                          * the 3x3 tile kernel and the persistent 1x1 / GEMM kernels */
	template<int POLICY = STORE_STREAM>
	__device__ inline void buffer_put(__amdgpu_buffer_rsrc_t rsrc, unsigned int byte_offset, unsigned int __attribute__((ext_vector_type(4))) words)
	{
		const u32x4_t v = { words.x, words.y, words.z, words.w };
		__builtin_amdgcn_raw_buffer_store_b128(v, rsrc, static_cast<int>(byte_offset), 0, POLICY);
	}
	template<int POLICY = STORE_STREAM>
	__device__ inline void buffer_put(__amdgpu_buffer_rsrc_t rsrc, unsigned int byte_offset, unsigned int __attribute__((ext_vector_type(2))) words)
	{
		const u32x2_t v = { words.x, words.y };
		__builtin_amdgcn_raw_buffer_store_b64(v, rsrc, static_cast<int>(byte_offset), 0, POLICY);
	}
	template<typename TE>
	__device__ inline uint4 splat_chunk(TE value, int valid)
	{
		constexpr int E = 16 / sizeof(TE);
		union
		{
			uint4 u;
			TE e[E];
		} t;
		t.u = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
		for (int i = 0; i < E; i++)
			if (i < valid)
				t.e[i] = value;
		return t.u;
	}

	constexpr int BLOCK_M = 128;
	constexpr int BLOCK_N = 128;
	constexpr int STEP_BYTES = 128; /* bytes of k consumed per operand row and step */
	constexpr int STEP_CHUNKS = STEP_BYTES / 16; /* 16-byte chunks per row and step */
	constexpr int FETCH_ROWS = 256 / STEP_CHUNKS; /* rows covered by one pass of the 256 work-items */
	constexpr int FETCH_PASSES = BLOCK_M / FETCH_ROWS; /* chunks of each operand a work-item fetches per step */
	constexpr int LDS_ROW = STEP_BYTES + 16; /* padded row pitch in LDS */
	constexpr int LDS_TILE = BLOCK_M * LDS_ROW; /* bytes of one operand tile */
	constexpr int LDS_BYTES = 4 * LDS_TILE; /* A and B, double buffered */

	/*
	 * Runs the k loop for one 128 x 128 output tile.
	 *
	 * A loader hands out the operand in k order: load(q, part) returns the 16-byte chunk `part` (0..7) of the current
	 * 128-byte k-slice of tile row (t / 8 + 32 * q), q = 0..3, where t is the calling work-item (zeros outside the matrix
	 * and for any k-slice at or past `steps`: the pipeline reads up to three slices beyond the end), and next() moves to the
	 * following k-slice.  Work-item t therefore fetches chunk (t % 8) of four rows of each operand.
	 *
	 * Software pipeline, iteration s (register sets R0 / R1 alternate, LDS buffers L0 / L1 alternate):
	 *     barrier
	 *     R[s % 2]   <- global(s + 2)             two k-slices ahead of the MFMAs
	 *     MFMAs of slice s from L[s % 2]
	 *     L[(s+1) % 2] <- R[(s+1) % 2]            slice s + 1, fetched during iteration s - 1
	 * so a global load has the MFMAs of two iterations (2 x 16 x 32 cycles per wavefront) to land before it is needed.
	 * acc[tm][tn] is the (tm, tn) 32 x 32 tile of this wavefront's 64 x 64 quadrant.
	 */
	template<typename TE, typename LoadA, typename LoadB>
	__device__ __forceinline__ void block_mma(char *lds, int steps, LoadA &load_a, LoadB &load_b, typename Mma<TE>::acc_t (&acc)[2][2])
	{
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wm = wave >> 1, wn = wave & 1;
		const int fpart = tid & (STEP_CHUNKS - 1);
		const int st_off = (tid / STEP_CHUNKS) * LDS_ROW + fpart * 16;
		const int rd_a = (wm * 64 + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;
		const int rd_b = (wn * 64 + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;

#pragma unroll
		for (int i = 0; i < 2; i++)
#pragma unroll
			for (int j = 0; j < 2; j++)
#pragma unroll
				for (int v = 0; v < 16; v++)
					acc[i][j][v] = 0;
		if (steps <= 0)
			return;

		uint4 ra[2][FETCH_PASSES], rb[2][FETCH_PASSES];
		auto fetch = [&](uint4 (&a)[FETCH_PASSES], uint4 (&b)[FETCH_PASSES])
		{
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				a[q] = load_a.load(q, fpart);
				b[q] = load_b.load(q, fpart);
			}
			load_a.next();
			load_b.next();
		};
		auto stash = [&](int buffer, const uint4 (&a)[FETCH_PASSES], const uint4 (&b)[FETCH_PASSES])
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
		auto multiply = [&](int buffer)
		{
			const char *sa = lds + buffer * 2 * LDS_TILE;
			const char *sb = sa + LDS_TILE;
			constexpr int SLABS = STEP_BYTES / 32;
			Chunk a[2][2], b[2][2]; /* operands of two consecutive 32-byte slabs: LDS reads run one slab ahead of the MFMAs */
			auto read = [&](int slab, Chunk (&ra_)[2], Chunk (&rb_)[2])
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
				/* a wavefront with operands in hand goes ahead of one that is still issuing loads (measured: helps the short 16-bit
				 * and int8 MFMAs, hurts the sixteen-pass fp32 ones, whose loaders then starve) */
				if (sizeof(TE) < 4)
					burst_priority(slab);
#pragma unroll
				for (int i = 0; i < 2; i++)
#pragma unroll
					for (int j = 0; j < 2; j++)
						Mma<TE>::run(a[slab & 1][i], b[slab & 1][j], acc[i][j]);
				if (sizeof(TE) < 4 && slab + 1 == SLABS)
					__builtin_amdgcn_s_setprio(0);
			}
		};

		/* The loop body is branch-free on purpose: the step count is rounded up to even and the loaders return zeros past
		 * the last k-slice, so the register sets and wait counts are the same in every iteration and a load issued in one
		 * half-iteration is only waited for one and a half iterations later. */
		fetch(ra[0], rb[0]);
		fetch(ra[1], rb[1]);
		stash(0, ra[0], rb[0]);
		for (int s = 0; s < steps; s += 2)
		{
			__syncthreads();
			fetch(ra[0], rb[0]);
			multiply(0);
			stash(1, ra[1], rb[1]);
			__syncthreads();
			fetch(ra[1], rb[1]);
			multiply(1);
			stash(0, ra[0], rb[0]);
		}
	}

	/*
	 * Hands an accumulator tile to the epilogue in row-major order.  The workgroup's tile is (2 * TM * 32) rows by 128
	 * columns when its four wavefronts form a 2 x 2 grid (WAVES_N = 2, wavefront tile TM*32 x 64), or (4 * TM * 32) rows by
	 * 64 columns when they are stacked (WAVES_N = 1).  The accumulators go through LDS in TM passes so that afterwards each
	 * work-item owns 4 consecutive columns of a row and neighbouring work-items cover a whole row: global stores are
	 * contiguous rows.  A work-item always gets the same 4 columns (drain_column()), so per-column constants can be loaded
	 * once, up front.  f(row, v, slot) is called with the tile-relative row, the CPL accumulators v[0..CPL-1] (CPL = 4 unless the
 * caller asks for 8 or 16 columns per work-item, which makes 16-byte stores of 2-byte and 1-byte outputs possible) and the
	 * number of the call (DrainRows<...>::row(slot) is that row: a caller can prefetch per-row data long before the drain).
	 * Must be called by all 256 work-items, after the last LDS read of the k loop; `lds` needs drain_bytes<WAVES_N>().
	 */
	template<int WAVES_N, int CPL = 4> struct DrainShape
	{
		static constexpr int cols = 64 * WAVES_N; /* columns of the workgroup tile */
		static constexpr int pitch = cols + 4; /* words per LDS row: keeps rows 16-byte aligned and staggers banks */
		static constexpr int rows_per_pass = 32 * (4 / WAVES_N); /* one 32-row MFMA tile of every wavefront row */
		static constexpr int threads_per_row = cols / CPL; /* CPL: consecutive columns handed to one work-item (4, 8 or 16) */
		static constexpr int bytes = rows_per_pass * pitch * 4;
	};
	template<int WAVES_N, int CPL = 4>
	__device__ inline int drain_column()
	{
		return (threadIdx.x % DrainShape<WAVES_N, CPL>::threads_per_row) * CPL;
	}
	/* The rows a work-item is handed by drain_tile, in the order of its calls: slot = tm * iterations + it. */
	template<int TM, int WAVES_N, int CPL = 4> struct DrainRows
	{
		typedef DrainShape<WAVES_N, CPL> D;
		static constexpr int row_step = 256 / D::threads_per_row; /* rows covered by one sweep of the workgroup */
		static constexpr int iterations = D::rows_per_pass / row_step;
		static constexpr int slots = TM * iterations;
		__device__ static inline int row(int slot)
		{
			const int tm = slot / iterations, it = slot - tm * iterations;
			const int rl = threadIdx.x / D::threads_per_row + it * row_step; /* row within the pass */
			return (rl >> 5) * (TM * 32) + tm * 32 + (rl & 31);
		}
	};
	/* `before_pass(tm)` runs ahead of the LDS hand-over of pass tm: the place to request per-row data (a residual) whose
	 * latency the hand-over then hides */
	template<typename TE, int TM, int WAVES_N, int CPL = 4, typename F, typename P>
	__device__ __forceinline__ void drain_tile(char *lds, const typename Mma<TE>::acc_t (&acc)[TM][2], const F &f, const P &before_pass)
	{
		typedef typename Mma<TE>::scalar_t S;
		typedef DrainShape<WAVES_N, CPL> D;
		static_assert(sizeof(S) == 4, "accumulators are 32-bit");
		static_assert(CPL == 4 || CPL == 8 || CPL == 16, "a work-item takes 4, 8 or 16 consecutive columns");
		S *sm = reinterpret_cast<S*>(lds);
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wm = WAVES_N == 2 ? (wave >> 1) : wave;
		const int wn = WAVES_N == 2 ? (wave & 1) : 0;
		const int col = drain_column<WAVES_N, CPL>();
		constexpr int ROW_STEP = 256 / D::threads_per_row; /* rows covered by one sweep of the workgroup */
#pragma unroll
		for (int tm = 0; tm < TM; tm++)
		{
			before_pass(tm);
			__syncthreads();
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
#pragma unroll
				for (int i = 0; i < 4; i++)
#pragma unroll
					for (int j = 0; j < 4; j++)
						sm[(wm * 32 + 8 * i + 4 * (lane >> 5) + j) * D::pitch + wn * 64 + tn * 32 + (lane & 31)] = acc[tm][tn][4 * i + j];
			__syncthreads();
			/* all LDS reads of the pass first, then the stores: the reads are independent and overlap */
			constexpr int ITERS = D::rows_per_pass / ROW_STEP;
			typedef S quad_t __attribute__((ext_vector_type(4))); /* a true vector type keeps the 16-byte LDS reads whole */
			quad_t vals[ITERS][CPL / 4];
#pragma unroll
			for (int it = 0; it < ITERS; it++)
#pragma unroll
				for (int part = 0; part < CPL / 4; part++)
					vals[it][part] = *reinterpret_cast<const quad_t*>(sm + (tid / D::threads_per_row + it * ROW_STEP) * D::pitch + col + 4 * part);
#pragma unroll
			for (int it = 0; it < ITERS; it++)
			{
				S v[CPL];
#pragma unroll
				for (int q = 0; q < CPL; q++)
					v[q] = vals[it][q / 4][q % 4];
				f(DrainRows<TM, WAVES_N, CPL>::row(tm * ITERS + it), v, tm * ITERS + it);
			}
		}
	}

	template<typename TE, int TM, int WAVES_N, int CPL = 4, typename F>
	__device__ __forceinline__ void drain_tile(char *lds, const typename Mma<TE>::acc_t (&acc)[TM][2], const F &f)
	{
		drain_tile<TE, TM, WAVES_N, CPL>(lds, acc, f, [](int) {});
	}
	/*
	 * The same hand-over for epilogues that are long (a switch over nine activation functions with their exponentials and
	 * logarithms): the rows of a pass are walked by a loop that stays a loop, so the epilogue is instantiated once per pass
	 * instead of once per row, while the passes themselves are written out, so that every index into the accumulators is
	 * a constant.  (With one unrollable loop nest the compiler gave up unrolling at that size, the accumulator indices became
	 * variables and the accumulators lived in scratch memory for the whole kernel.)
	 */
	template<typename TE, int TM, int WAVES_N, typename F>
	__device__ __forceinline__ void drain_tile_rolled(char *lds, const typename Mma<TE>::acc_t (&acc)[TM][2], const F &f)
	{
		static_assert(TM == 1 || TM == 2, "one or two passes, written out");
		typedef typename Mma<TE>::scalar_t S;
		typedef DrainShape<WAVES_N, 4> D;
		S *sm = reinterpret_cast<S*>(lds);
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wm = WAVES_N == 2 ? (wave >> 1) : wave;
		const int wn = WAVES_N == 2 ? (wave & 1) : 0;
		const int col = drain_column<WAVES_N, 4>();
		constexpr int ROW_STEP = 256 / D::threads_per_row;
		constexpr int ITERS = D::rows_per_pass / ROW_STEP;
		auto pass = [&](auto which) __attribute__((always_inline))
		{
			constexpr int tm = decltype(which)::value;
			__syncthreads();
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
#pragma unroll
				for (int i = 0; i < 4; i++)
#pragma unroll
					for (int j = 0; j < 4; j++)
						sm[(wm * 32 + 8 * i + 4 * (lane >> 5) + j) * D::pitch + wn * 64 + tn * 32 + (lane & 31)] = acc[tm][tn][4 * i + j];
			__syncthreads();
#pragma unroll 1
			for (int it = 0; it < ITERS; it++)
			{
				typedef S quad_t __attribute__((ext_vector_type(4)));
				const quad_t q = *reinterpret_cast<const quad_t*>(sm + (tid / D::threads_per_row + it * ROW_STEP) * D::pitch + col);
				const S v[4] = { q[0], q[1], q[2], q[3] };
				f(DrainRows<TM, WAVES_N, 4>::row(tm * ITERS + it), v, tm * ITERS + it);
			}
		};
		pass(std::integral_constant<int, 0>());
		if constexpr (TM == 2)
			pass(std::integral_constant<int, 1>());
	}
	/*
	 * The same hand-over for workgroups whose four wavefronts are stacked (each owns TM 32-row tiles by 64 columns, the
	 * workgroup (4 * TM * 32) rows by 64 columns), without workgroup barriers after the first: a wavefront passes its own
	 * accumulators through its own 8.5 KB of LDS, where its writes and reads stay in program order, so nobody waits for the
	 * slowest wavefront between the passes.  A work-item gets CPL consecutive columns (drain_column<1, CPL>()) of rows of its
	 * own wavefront; PrivateDrainRows<...>::row(slot) names the row of call `slot`.  `lds` needs 4 * PrivateDrainRows::bytes.
	 */
	template<int TM, int CPL> struct PrivateDrainRows
	{
		static constexpr int pitch = 64 + 4; /* words per LDS row: keeps rows 16-byte aligned and staggers banks */
		static constexpr int threads_per_row = 64 / CPL;
		static constexpr int rows_per_sweep = 64 / threads_per_row; /* rows one wavefront covers per instruction */
		static constexpr int iterations = 32 / rows_per_sweep; /* sweeps per 32-row MFMA tile */
		static constexpr int slots = TM * iterations;
		static constexpr int bytes = 32 * pitch * 4; /* per wavefront */
		__device__ static inline int row(int slot)
		{
			const int tm = slot / iterations, it = slot - tm * iterations;
			const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
			return wave * (TM * 32) + tm * 32 + lane / threads_per_row + it * rows_per_sweep;
		}
	};
	template<typename TE, int TM, int CPL, typename F>
	__device__ __forceinline__ void drain_tile_private(char *lds, const typename Mma<TE>::acc_t (&acc)[TM][2], const F &f)
	{
		typedef typename Mma<TE>::scalar_t S;
		typedef PrivateDrainRows<TM, CPL> D;
		static_assert(sizeof(S) == 4, "accumulators are 32-bit");
		static_assert(CPL == 4 || CPL == 8 || CPL == 16, "a work-item takes 4, 8 or 16 consecutive columns");
		const int lane = threadIdx.x & 63;
		const int wave = threadIdx.x >> 6;
		S *sm = reinterpret_cast<S*>(lds + wave * D::bytes);
		const int col = (lane % D::threads_per_row) * CPL;
		__syncthreads(); /* the last LDS reads of the k loop, by any wavefront, are over */
#pragma unroll
		for (int tm = 0; tm < TM; tm++)
		{
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
#pragma unroll
				for (int i = 0; i < 4; i++)
#pragma unroll
					for (int j = 0; j < 4; j++)
						sm[(8 * i + 4 * (lane >> 5) + j) * D::pitch + tn * 32 + (lane & 31)] = acc[tm][tn][4 * i + j];
			/* what other lanes of this wavefront wrote is read next: LDS serves a wavefront's accesses in order, the fence keeps
			 * the compiler from reordering them */
			__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
			/* read back as 16-byte vectors (a true vector type: a struct of four is taken apart by the compiler and put back
			 * together as 12 + 8 + 8 + 4 bytes) */
			typedef S quad_t __attribute__((ext_vector_type(4)));
			quad_t vals[D::iterations][CPL / 4];
#pragma unroll
			for (int it = 0; it < D::iterations; it++)
#pragma unroll
				for (int part = 0; part < CPL / 4; part++)
					vals[it][part] = *reinterpret_cast<const quad_t*>(sm + (lane / D::threads_per_row + it * D::rows_per_sweep) * D::pitch + col + 4 * part);
			__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront"); /* the next pass overwrites what was just read */
#pragma unroll
			for (int it = 0; it < D::iterations; it++)
			{
				S v[CPL];
#pragma unroll
				for (int q = 0; q < CPL; q++)
					v[q] = vals[it][q / 4][q % 4];
				f(D::row(tm * D::iterations + it), v, tm * D::iterations + it);
			}
		}
	}
}

#endif /* AVHIP_MFMA_CORE_HPP_ */
