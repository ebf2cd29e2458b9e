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
 *   one k-step consumes 64 bytes of every operand row (32 fp16/bf16, 64 int8, 16 fp32 values);
 *   per step each work-item moves two 16-byte chunks of A and two of B: global -> registers -> LDS, the global loads of
 *   step s+1 are issued before the MFMAs of step s (register prefetch) and LDS is double buffered, so there is one
 *   barrier per step;
 *   LDS rows are padded from 64 to 80 bytes so that the 32 rows a wavefront reads with one ds_read_b128 spread over banks.
 * MFMA shapes: v_mfma_f32_32x32x16_{f16,bf16}, v_mfma_i32_32x32x32_i8, v_mfma_f32_32x32x2_f32 (four per 16-byte chunk).
 * Lane l of a wavefront supplies row (l % 32) of the operand tile and the k-chunk (l / 32); it receives, for output column
 * (l % 32), the 16 rows 8*i + 4*(l / 32) + j (i, j < 4).
 */
#ifndef AVHIP_MFMA_CORE_HPP_
#define AVHIP_MFMA_CORE_HPP_

#include "common.hpp"

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
	};
	template<> struct Mma<f16_t>
	{
		typedef f32x16_t acc_t;
		typedef float scalar_t;
		__device__ static inline void run(const Chunk &a, const Chunk &b, acc_t &c)
		{
			c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.hf, b.hf, c, 0, 0, 0);
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
	constexpr int STEP_BYTES = 64; /* bytes of k consumed per row and step */
	constexpr int LDS_ROW = 80; /* padded row pitch in LDS */
	constexpr int LDS_TILE = BLOCK_M * LDS_ROW; /* bytes of one operand tile */
	constexpr int LDS_BYTES = 4 * LDS_TILE; /* A and B, double buffered */

	/*
	 * Runs the k loop for one 128 x 128 output tile.
	 *   LoadA(step, q, part) / LoadB(step, q, part) return the 16-byte chunk `part` (0..3) of the 64-byte k-slice `step` of
	 *   tile row / tile column (t / 4 + 64 * q), q = 0 or 1, where t is the calling work-item; zeros outside the matrix.
	 * Work-item t thus fetches chunk (t % 4) of rows (t / 4) and (t / 4 + 64) of both operands.
	 * acc[tm][tn] is the (tm, tn) 32 x 32 tile of this wavefront's 64 x 64 quadrant.
	 */
	template<typename TE, typename LoadA, typename LoadB>
	__device__ inline void block_mma(char *lds, int steps, const LoadA &load_a, const LoadB &load_b, typename Mma<TE>::acc_t (&acc)[2][2])
	{
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wm = wave >> 1, wn = wave & 1;
		const int frow = tid >> 2, fpart = tid & 3;

#pragma unroll
		for (int i = 0; i < 2; i++)
#pragma unroll
			for (int j = 0; j < 2; j++)
#pragma unroll
				for (int v = 0; v < 16; v++)
					acc[i][j][v] = 0;

		uint4 ra[2], rb[2];
		if (steps > 0)
		{
			ra[0] = load_a(0, 0, fpart);
			ra[1] = load_a(0, 1, fpart);
			rb[0] = load_b(0, 0, fpart);
			rb[1] = load_b(0, 1, fpart);
		}
		const int st_off = frow * LDS_ROW + fpart * 16;
		const int rd_a = (wm * 64 + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;
		const int rd_b = (wn * 64 + (lane & 31)) * LDS_ROW + (lane >> 5) * 16;

		for (int step = 0; step < steps; step++)
		{
			char *sa = lds + (step & 1) * 2 * LDS_TILE;
			char *sb = sa + LDS_TILE;
			*reinterpret_cast<uint4*>(sa + st_off) = ra[0];
			*reinterpret_cast<uint4*>(sa + st_off + 64 * LDS_ROW) = ra[1];
			*reinterpret_cast<uint4*>(sb + st_off) = rb[0];
			*reinterpret_cast<uint4*>(sb + st_off + 64 * LDS_ROW) = rb[1];
			__syncthreads();
			if (step + 1 < steps)
			{
				ra[0] = load_a(step + 1, 0, fpart);
				ra[1] = load_a(step + 1, 1, fpart);
				rb[0] = load_b(step + 1, 0, fpart);
				rb[1] = load_b(step + 1, 1, fpart);
			}
#pragma unroll
			for (int slab = 0; slab < 2; slab++)
			{
				Chunk a[2], b[2];
#pragma unroll
				for (int i = 0; i < 2; i++)
				{
					a[i].u = *reinterpret_cast<const uint4*>(sa + rd_a + i * 32 * LDS_ROW + slab * 32);
					b[i].u = *reinterpret_cast<const uint4*>(sb + rd_b + i * 32 * LDS_ROW + slab * 32);
				}
#pragma unroll
				for (int i = 0; i < 2; i++)
#pragma unroll
					for (int j = 0; j < 2; j++)
						Mma<TE>::run(a[i], b[j], acc[i][j]);
			}
		}
	}

	/*
	 * Hands the 128 x 128 accumulator tile to the epilogue in row-major order: the accumulators go through LDS (reusing the
	 * operand buffers, in two halves of 64 rows) so that afterwards each work-item owns 4 consecutive columns of a row and
	 * 32 neighbouring work-items cover one 128-column row, i.e. global stores are whole contiguous rows.
	 * f(row, col, v) is called with tile-relative row (0..127), col (multiple of 4) and the four accumulators v[0..3].
	 * Must be called by all 256 work-items after block_mma.
	 */
	constexpr int DRAIN_PITCH = 132; /* words per LDS row: 128 + 4 keeps rows 16-byte aligned and staggers banks */
	template<typename TE, typename F>
	__device__ inline void drain_tile(char *lds, const typename Mma<TE>::acc_t (&acc)[2][2], const F &f)
	{
		typedef typename Mma<TE>::scalar_t S;
		static_assert(sizeof(S) == 4 && 64 * DRAIN_PITCH * 4 <= LDS_BYTES, "drain buffer must fit the operand buffers");
		S *sm = reinterpret_cast<S*>(lds);
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
		for (int tm = 0; tm < 2; tm++)
		{
			__syncthreads();
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
#pragma unroll
				for (int i = 0; i < 4; i++)
#pragma unroll
					for (int j = 0; j < 4; j++)
						sm[(wm * 32 + 8 * i + 4 * (lane >> 5) + j) * DRAIN_PITCH + wn * 64 + tn * 32 + (lane & 31)] = acc[tm][tn][4 * i + j];
			__syncthreads();
			for (int e = tid; e < 64 * 32; e += 256)
			{
				const int rl = e >> 5;
				const int col = (e & 31) * 4;
				const int row = (rl >> 5) * 64 + tm * 32 + (rl & 31);
				const Pack<S, 4> p = *reinterpret_cast<const Pack<S, 4>*>(sm + rl * DRAIN_PITCH + col);
				f(row, col, p.v);
			}
		}
	}
}

#endif /* AVHIP_MFMA_CORE_HPP_ */
