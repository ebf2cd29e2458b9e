/*
 * conv_pointwise_block.hip -- 1x1 convolution of 16-bit tensors with many filters (the channel-mixing layers of a network) as a
 * GEMM whose pixel operand is resident in LDS for the whole k walk and whose filters come to the matrix cores straight from L2.
 *
 * Same arithmetic as the implicit-GEMM forward of the reference (src/conv2d_implicit_gemm.cu:152-301, entry point
 * cuda_convolution2dImplicitGemm, :303) for a 1x1 filter: y[p][k] = act(alpha1 * sum_c x[p][c] * w[k][c] + bias[k] + alpha2 * z[p][k]).
 * With k = C of 128..256 an output element costs half an MFMA clock, so what decides is everything around the MFMAs; here
 *
 *   workgroup = 8 wavefronts = a block of up to 224 consecutive pixels (GEMM rows; 1x1, stride 1, no padding: the rows of x are
 *               the rows of the GEMM) x 512 filters.  The block's pixels, all channels, are fetched once into LDS (row pitch
 *               2C + 16 bytes: conflict-free 16-byte reads of 32 consecutive rows); ONE barrier in the kernel;
 *   wavefront w owns filters 64w .. 64w + 63 for all rows: two filter tiles of 32, taken over the rows in two passes of 4 and 3
 *               MFMA row tiles (128 accumulator registers at most).  Its filter operand comes from global memory (L2) in MFMA
 *               register layout, written that way once per weight tensor by avhip_conv2d_pointwise_block_weight_layout:
 *               [tile of 32 filters][16-channel slab][lane][16 bytes], through a ring of register sets;
 *   epilogue  : no barrier.  Filters are the rows of the MFMA tile, so a lane holds runs of four consecutive filters of one
 *               pixel; bias, residual, activation and rounding happen there, the rounded runs of a row tile pass through the
 *               wavefront's own 4.5 KB of LDS and leave as whole 128-byte lines of y (a wavefront's 64 filters are one line of
 *               every pixel), written through as the kernel runs;
 *   wavefronts 0-3 take the passes in the order (rows 0-127, rows 128-223), wavefronts 4-7 the other way round: the two
 *               wavefronts that share a SIMD are then in different parts of their work, one multiplying while the other
 *               stores, and nothing but the one barrier ever makes them wait for each other.
 * Limits: fp16 / bf16, 1x1, stride 1, dilation 1, no padding, C = 128 or 256, K a multiple of 512, beta = 0, LINEAR or RELU,
 * tensors below 2 GiB.
 */
#include <atomic>

#include "conv_epilogue.hpp"
#include "mfma_core.hpp"

#ifdef POINTWISE_BLOCK_STAMPS
__device__ unsigned long long g_block_stamps[4096 * 8];
#define BSTAMP(i) do { if (threadIdx.x == 0) g_block_stamps[(blockIdx.x % 4096) * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
extern "C" __attribute__((visibility("default"))) int avhip_debug_block_stamps(void *out)
{
	return static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_block_stamps), sizeof(g_block_stamps)));
}
#else
#define BSTAMP(i) do { } while (0)
#endif

#ifndef POINTWISE_BLOCK_STORE_POLICY
#define POINTWISE_BLOCK_STORE_POLICY 19 /* sc0 sc1 nt: whole lines, written through as the kernel runs */
#endif
#ifndef POINTWISE_BLOCK_B_RING
#define POINTWISE_BLOCK_B_RING 4
#endif

namespace
{
	using namespace avhip;

	constexpr int P_THREADS = 512;
	constexpr int P_ROW_TILES = 7; /* MFMA tiles of 32 GEMM rows per workgroup: passes of 4 and 3 */
	constexpr int P_ROWS = P_ROW_TILES * 32;
	constexpr int P_FIRST_TILES = 4;
	constexpr int P_FILTERS = 512; /* per workgroup: 8 wavefronts x 2 tiles of 32 */
	constexpr int P_OPERAND = 1024; /* one MFMA operand of a wavefront: 64 lanes x 16 bytes */

	struct BlockGeom
	{
		int M; /* pixels: N * H * W */
		int K;
		int rows; /* pixels per workgroup */
		int filter_tiles; /* K / 32 */
	};

	/* Weights in MFMA operand layout: one work-item = one lane's 16 bytes of (tile of 32 filters, slab of 16 channels). */
	template<typename TE>
	__global__ void k_pointwise_block_weight_layout(const TE *__restrict__ w, uint4 *__restrict__ U, int K, int C, int slabs, int filter_tiles)
	{
		const int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
		const int64_t total = static_cast<int64_t>(filter_tiles) * slabs * 64;
		if (e >= total)
			return;
		const int lane = static_cast<int>(e & 63);
		const int64_t t = e >> 6;
		const int slab = static_cast<int>(t % slabs);
		const int tile = static_cast<int>(t / slabs);
		const int k = tile * 32 + (lane & 31);
		const int c0 = slab * 16 + (lane >> 5) * 8;
		union
		{
			uint4 u;
			TE e[8];
		} out;
		out.u = make_uint4(0u, 0u, 0u, 0u);
		if (k < K)
		{
#pragma unroll
			for (int q = 0; q < 8; q++)
				if (c0 + q < C)
					out.e[q] = w[static_cast<int64_t>(k) * C + c0 + q];
		}
		U[e] = out.u;
	}

	template<typename TE, int SLABS>
	__global__ __launch_bounds__(P_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_pointwise_block(const TE *__restrict__ x, const void *__restrict__ U,
			BlockGeom g, FloatEpilogue<TE> epi)
	{
		constexpr unsigned int SZ = sizeof(TE);
		constexpr int ROW_BYTES = SLABS * 16 * static_cast<int>(SZ);
		constexpr int PITCH = ROW_BYTES + 16;
		constexpr int CHUNKS_PER_ROW = ROW_BYTES / 16;
		constexpr int SWEEP_ROWS = P_THREADS / CHUNKS_PER_ROW; /* rows one round of loads of the workgroup covers */
		constexpr int SWEEPS = P_ROWS / SWEEP_ROWS;
		/* behind the pixels: one region per wavefront, [32 pixels][its 64 filters as stored + 16 bytes], through which a row tile's
		 * results change from the layout of the accumulators to whole lines of y */
		constexpr int OUT_PITCH = 64 * static_cast<int>(SZ) + 16, OUT_BYTES = 32 * OUT_PITCH, X_BYTES = P_ROWS * PITCH;
		static_assert(P_ROWS % SWEEP_ROWS == 0 && X_BYTES + (P_THREADS / 64) * OUT_BYTES <= 160 * 1024, "whole sweeps; LDS of a compute unit");
		__shared__ __attribute__((aligned(16))) char lds[X_BYTES + (P_THREADS / 64) * OUT_BYTES];
		BSTAMP(0);
		epi.pin();
		keep_in_sgpr(g.M);
		keep_in_sgpr(g.K);
		keep_in_sgpr(g.rows);
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		/* the filter blocks of a pixel block follow each other on one XCD, whose L2 then holds the pixels for the second one */
		unsigned int block = blockIdx.x, filter_block = 0;
		if (gridDim.y != 1)
			xcd_tile(block, filter_block);
		const int kb = static_cast<int>(filter_block);
		const int row0 = static_cast<int>(block) * g.rows;
		const int rows = g.M - row0 < g.rows ? g.M - row0 : g.rows; /* real pixels of this block */

		/* the block's pixels: work-item t takes 16-byte chunk t % CHUNKS_PER_ROW of rows t / CHUNKS_PER_ROW + k * SWEEP_ROWS; rows
		 * past the block's last are zeros (out-of-range offsets) */
		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, static_cast<unsigned int>(g.M) * ROW_BYTES);
		const int l_row = tid / CHUNKS_PER_ROW, l_chunk = tid % CHUNKS_PER_ROW;
		uint4 raw[SWEEPS];
#pragma unroll
		for (int k = 0; k < SWEEPS; k++)
		{
			const int r = l_row + k * SWEEP_ROWS;
			const unsigned int offset = r < rows ? static_cast<unsigned int>(row0 + r) * ROW_BYTES + l_chunk * 16 : OUT_OF_RANGE;
			const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rx, static_cast<int>(offset), 0, 0);
			raw[k] = make_uint4(v[0], v[1], v[2], v[3]);
		}

		/* filter operand: slab s of this wavefront's two tiles, a kilobyte each */
		const __amdgpu_buffer_rsrc_t ru = make_buffer(U, static_cast<unsigned int>(g.filter_tiles) * SLABS * P_OPERAND);
		const unsigned int b_offset = static_cast<unsigned int>(((kb * (P_FILTERS / 32) + wave * 2) * SLABS) * P_OPERAND + lane * 16);
		constexpr int B_RING = POINTWISE_BLOCK_B_RING, B_AHEAD = B_RING - 1;
		static_assert(SLABS % B_RING == 0, "the filter ring stands at 0 when a pass starts");
		Chunk bq[B_RING][2];
		auto load_b = [&](int slab, Chunk (&set)[2]) __attribute__((always_inline)) /* slab of either pass: both walk the same filters */
		{
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
			{
				const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(ru, static_cast<int>(b_offset), (tn * SLABS + slab % SLABS) * P_OPERAND, 0);
				set[tn].u = make_uint4(v[0], v[1], v[2], v[3]);
			}
		};
#pragma unroll
		for (int s = 0; s < B_AHEAD; s++)
			load_b(s, bq[s]);

		/* into LDS; the one barrier */
		{
			int l_base = l_row * PITCH + l_chunk * 16;
			asm volatile("" : "+v"(l_base));
			int l_far = l_base + (SWEEPS / 2) * SWEEP_ROWS * PITCH; /* offsets beyond 64 KB do not fit the instruction's immediate */
			asm volatile("" : "+v"(l_far));
#pragma unroll
			for (int k = 0; k < SWEEPS; k++)
			{
				if (k < SWEEPS / 2)
					*reinterpret_cast<uint4*>(lds + l_base + k * SWEEP_ROWS * PITCH) = raw[k];
				else
					*reinterpret_cast<uint4*>(lds + l_far + (k - SWEEPS / 2) * SWEEP_ROWS * PITCH) = raw[k];
			}
		}
		BSTAMP(1);
		__syncthreads();
		BSTAMP(2);

		/* pixel operand address: lane l supplies GEMM row (l % 32) of a 32-row tile and the 8-channel half (l / 32) of a slab */
		const int a_lane = (lane & 31) * PITCH + (lane >> 5) * 16;
		const __amdgpu_buffer_rsrc_t ry = make_buffer(epi.y, static_cast<unsigned int>(g.M) * g.K * SZ);
		const __amdgpu_buffer_rsrc_t rz = make_buffer(epi.z, epi.z != nullptr ? static_cast<unsigned int>(g.M) * g.K * SZ : 0u);
		const bool relu = epi.activation == ACT_RELU, has_z = epi.z != nullptr;
		const int kcol = kb * P_FILTERS + wave * 64; /* this wavefront's first filter */
		typedef float f32x4 __attribute__((ext_vector_type(4)));

		constexpr int A_RING = 8, A_AHEAD = 6;
		/* One pass: NT row tiles from GEMM row `first_row` on.  FRESH: nothing of this pass could be requested ahead. */
		auto run_pass = [&](auto nt_tag, int first_row, bool prefetch_next) __attribute__((always_inline))
		{
			constexpr int NT = decltype(nt_tag)::value;
			constexpr int CHUNKS = SLABS * NT;
			static_assert(CHUNKS % A_RING == 0, "the pixel ring stands at 0 when a pass starts");
			int a_base = first_row * PITCH + a_lane;
			asm volatile("" : "+v"(a_base));
			typename Mma<TE>::acc_t acc[NT][2];
			Chunk a[A_RING];
			auto read_a = [&](int c, Chunk &dst) __attribute__((always_inline)) /* chunk = (slab, row tile) in the order of use */
			{
				dst.u = *reinterpret_cast<const uint4*>(lds + a_base + (c % NT) * 32 * PITCH + (c / NT) * 32);
			};
#pragma unroll
			for (int c = 0; c < A_AHEAD; c++)
				read_a(c, a[c]);
#pragma unroll
			for (int s = 0; s < SLABS; s++)
			{
				__builtin_amdgcn_sched_barrier(0);
				/* past the pass's last slab the ring asks for the first slabs again: the other pass walks the same filters */
				if (s + B_AHEAD < SLABS || prefetch_next)
					load_b(s + B_AHEAD, bq[(s + B_AHEAD) % B_RING]);
#pragma unroll
				for (int rt = 0; rt < NT; rt++)
				{
					const int c = s * NT + rt;
					if (c + A_AHEAD < CHUNKS)
						read_a(c + A_AHEAD, a[(c + A_AHEAD) % A_RING]);
#pragma unroll
					for (int tn = 0; tn < 2; tn++)
					{
						if (s == 0)
							Mma<TE>::start(bq[s % B_RING][tn], a[c % A_RING], acc[rt][tn]);
						else
							Mma<TE>::run(bq[s % B_RING][tn], a[c % A_RING], acc[rt][tn]);
					}
				}
				__builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
#pragma unroll
				for (int rt = 0; rt < NT; rt++)
				{
					__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
					__builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
				}
			}
			__builtin_amdgcn_sched_barrier(0);

			/* Out: accumulator registers 4i .. 4i + 3 of tile (rt, tn) are filters kcol + 32 tn + 8i + 4 (lane / 32) + 0..3 of pixel
			 * first_row + 32 rt + lane % 32.  Bias, residual, activation and the one rounding are applied in that layout; the rounded
			 * runs of a row tile then pass through this wavefront's own region of LDS (no barrier: LDS serves a wavefront's
			 * operations in order) and leave as whole 128-byte lines, eight lanes per pixel. */
			const int half = lane >> 5;
			int out_put = X_BYTES + wave * OUT_BYTES + (lane & 31) * OUT_PITCH + 4 * half * static_cast<int>(SZ);
			asm volatile("" : "+v"(out_put));
			int out_get = X_BYTES + wave * OUT_BYTES + (lane >> 3) * OUT_PITCH + (lane & 7) * 16;
			asm volatile("" : "+v"(out_get));
			auto leave = [&](auto with_relu, auto with_z) __attribute__((always_inline))
			{
				constexpr bool RELU = decltype(with_relu)::value, HAS_Z = decltype(with_z)::value;
				const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(epi.bias), 0, epi.bias != nullptr ? g.K * 4 : 0, 0x00020000);
				/* bias of this lane's four filters in every run: requested once per pass, behind the last MFMA */
				f32x4 bias[2][4];
#pragma unroll
				for (int tn = 0; tn < 2; tn++)
#pragma unroll
					for (int i = 0; i < 4; i++)
						bias[tn][i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rb, (kcol + 32 * tn + 8 * i + 4 * half) * 4, 0, 0));
				/* The residual in the layout of the accumulators: runs (2 pair, 2 pair + 1) of the two lanes of a pixel are 32
				 * consecutive bytes of z, fetched as 16 bytes per lane (the lower lane run 2 pair, the upper one run 2 pair + 1) and
				 * exchanged between the two by the swap.  One row tile ahead. */
				u32x4_t zr[2][2][2];
				auto request_z = [&](int rt, u32x4_t (&into)[2][2]) __attribute__((always_inline))
				{
					const int row = first_row + 32 * rt + (lane & 31);
#pragma unroll
					for (int tn = 0; tn < 2; tn++)
#pragma unroll
						for (int pair = 0; pair < 2; pair++)
						{
							const unsigned int offset = row < rows ? (static_cast<unsigned int>(row0 + row) * g.K + kcol + 32 * tn + 8 * (2 * pair + half)) * SZ
									: OUT_OF_RANGE;
							into[tn][pair] = __builtin_amdgcn_raw_buffer_load_b128(rz, static_cast<int>(offset), 0, 2);
						}
				};
				if (HAS_Z)
					request_z(0, zr[0]);
#pragma unroll
				for (int rt = 0; rt < NT; rt++)
				{
					if (HAS_Z && rt + 1 < NT)
						request_z(rt + 1, zr[(rt + 1) & 1]);
#pragma unroll
					for (int tn = 0; tn < 2; tn++)
#pragma unroll
						for (int pair = 0; pair < 2; pair++)
						{
							unsigned int zw[4] = { 0u, 0u, 0u, 0u };
							if (HAS_Z)
							{
								const u32x4_t &zq = zr[rt & 1][tn][pair];
								const auto s0 = __builtin_amdgcn_permlane32_swap(zq[0], zq[2], false, false);
								const auto s1 = __builtin_amdgcn_permlane32_swap(zq[1], zq[3], false, false);
								zw[0] = s0[0]; /* run 2 pair, this lane's half */
								zw[1] = s1[0];
								zw[2] = s0[1]; /* run 2 pair + 1 */
								zw[3] = s1[1];
							}
#pragma unroll
							for (int e = 0; e < 2; e++)
							{
								union
								{
									Pack<TE, 4> p;
									unsigned int w[2];
									uint2 u;
								} zin, out;
								zin.w[0] = zw[2 * e];
								zin.w[1] = zw[2 * e + 1];
#pragma unroll
								for (int q = 0; q < 4; q++)
								{
									float r = epi.alpha1 * acc[rt][tn][4 * (2 * pair + e) + q] + bias[tn][2 * pair + e][q];
									if (HAS_Z)
										r += epi.alpha2 * Traits<TE>::load(zin.p.v[q]);
									out.p.v[q] = Traits<TE>::store(RELU ? __builtin_fmaxf(r, 0.0f) : r);
								}
								*reinterpret_cast<uint2*>(lds + out_put + (32 * tn + 8 * (2 * pair + e)) * static_cast<int>(SZ)) = out.u;
							}
						}
					/* lane l: 16 bytes (l % 8) of pixel l / 8 + 8 it of the row tile */
#pragma unroll
					for (int it = 0; it < 4; it++)
					{
						const uint4 line = *reinterpret_cast<const uint4*>(lds + out_get + it * 8 * OUT_PITCH);
						const int row = first_row + 32 * rt + 8 * it + (lane >> 3);
						const unsigned int offset = row < rows ? (static_cast<unsigned int>(row0 + row) * g.K + kcol) * SZ + (lane & 7) * 16 : OUT_OF_RANGE;
						const u32x4_t words = { line.x, line.y, line.z, line.w };
						__builtin_amdgcn_raw_buffer_store_b128(words, ry, static_cast<int>(offset), 0, POINTWISE_BLOCK_STORE_POLICY);
					}
				}
			};
			if (relu && has_z)
				leave(std::true_type(), std::true_type());
			else if (relu)
				leave(std::true_type(), std::false_type());
			else if (has_z)
				leave(std::false_type(), std::true_type());
			else
				leave(std::false_type(), std::false_type());
		};
		if (wave < 4)
		{
			run_pass(std::integral_constant<int, P_FIRST_TILES>(), 0, true);
			BSTAMP(3);
			run_pass(std::integral_constant<int, P_ROW_TILES - P_FIRST_TILES>(), P_FIRST_TILES * 32, false);
		}
		else
		{
			run_pass(std::integral_constant<int, P_ROW_TILES - P_FIRST_TILES>(), P_FIRST_TILES * 32, true);
			run_pass(std::integral_constant<int, P_FIRST_TILES>(), 0, false);
		}
		BSTAMP(4);
	}

	/* Pixels per workgroup: the fewest rounds of workgroups over the compute units, then blocks of equal size. */
	int choose_block_rows(int64_t M, int filter_blocks)
	{
		const int64_t per_round = filter_blocks < 256 ? 256 / filter_blocks : 1; /* pixel blocks that run at once */
		const int64_t rounds = (M + P_ROWS * per_round - 1) / (P_ROWS * per_round);
		int64_t rows = (M + per_round * rounds - 1) / (per_round * rounds);
		rows = (rows + 3) / 4 * 4;
		return static_cast<int>(rows > P_ROWS ? P_ROWS : rows);
	}
	bool block_shape_ok(const avhipConvShape &s)
	{
		return s.R == 1 && s.S == 1 && s.stride_h == 1 && s.stride_w == 1 && s.pad_h == 0 && s.pad_w == 0 && s.Ho == s.H && s.Wo == s.W && (s.C == 128 || s.C == 256)
				&& s.K % P_FILTERS == 0 && s.K > 0 && s.N > 0 && s.H > 0 && s.W > 0;
	}
	std::atomic<int> block_mode { 1 };

	template<typename TE>
	int launch_block(hipStream_t st, const avhipConvShape &s, const void *x, const void *U, const void *bias, const void *z, void *y, double alpha1,
			double alpha2, int activation)
	{
		if (!aligned_to(x, 16) || !aligned_to(U, 16) || !aligned_to(y, 16) || (z != nullptr && !aligned_to(z, 16)) || (bias != nullptr && !aligned_to(bias, 16)))
			return AVHIP_NOT_SUPPORTED;
		const int64_t M = static_cast<int64_t>(s.N) * s.H * s.W;
		if (M * s.C * sizeof(TE) >= (1ll << 31) || M * s.K * sizeof(TE) >= (1ll << 31))
			return AVHIP_NOT_SUPPORTED;
		BlockGeom g;
		g.M = static_cast<int>(M);
		g.K = s.K;
		g.rows = choose_block_rows(M, s.K / P_FILTERS);
		g.filter_tiles = s.K / 32;
		const int64_t blocks = (M + g.rows - 1) / g.rows;
		if (blocks >= (1ll << 31) || s.K / P_FILTERS > 65535)
			return AVHIP_NOT_SUPPORTED;
		const FloatEpilogue<TE> epi { static_cast<const float*>(bias), static_cast<const TE*>(z), static_cast<TE*>(y), static_cast<float>(alpha1),
				static_cast<float>(alpha2), 0.0f, activation, s.K, true };
		const dim3 grid(static_cast<unsigned int>(blocks), static_cast<unsigned int>(s.K / P_FILTERS));
		if (s.C == 256)
			hipLaunchKernelGGL((k_pointwise_block<TE, 16>), grid, dim3(P_THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
		else
			hipLaunchKernelGGL((k_pointwise_block<TE, 8>), grid, dim3(P_THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
		return 0;
	}
}

extern "C" int avhip_set_pointwise_block(int mode)
{
	return mode < 0 ? block_mode.load() : block_mode.exchange(mode);
}

extern "C" int avhip_conv2d_pointwise_block_plan(int dtype, const avhipConvShape *shape, int *workgroups, int *rows_used)
{
	if (shape == nullptr)
		return AVHIP_BAD_PARAM;
	const avhipConvShape &s = *shape;
	if (block_mode.load() == 0 || (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16) || !block_shape_ok(s))
		return AVHIP_NOT_SUPPORTED;
	const int64_t M = static_cast<int64_t>(s.N) * s.H * s.W;
	const int rows = choose_block_rows(M, s.K / P_FILTERS);
	const int64_t groups = (M + rows - 1) / rows * (s.K / P_FILTERS);
	if (workgroups != nullptr)
		workgroups[0] = groups > 0x7FFFFFFF ? 0x7FFFFFFF : static_cast<int>(groups);
	if (rows_used != nullptr)
		rows_used[0] = rows;
	return 0;
}

extern "C" int64_t avhip_conv2d_pointwise_block_weight_bytes(int K, int C)
{
	if (K <= 0 || C <= 0)
		return 0;
	return static_cast<int64_t>((K + 31) / 32) * ((C + 15) / 16) * P_OPERAND;
}

extern "C" int avhip_conv2d_pointwise_block_weight_layout(void *stream, int dtype, const void *w, void *U, int K, int C)
{
	if (w == nullptr || U == nullptr || K <= 0 || C <= 0)
		return AVHIP_BAD_PARAM;
	const int slabs = (C + 15) / 16, tiles = (K + 31) / 32;
	const int64_t total = static_cast<int64_t>(tiles) * slabs * 64;
	const dim3 grid(ceil_div(total, 256));
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (dtype)
	{
		case DT_FLOAT16:
			hipLaunchKernelGGL((k_pointwise_block_weight_layout<f16_t>), grid, dim3(256), 0, st, static_cast<const f16_t*>(w), static_cast<uint4*>(U), K, C, slabs, tiles);
			return 0;
		case DT_BFLOAT16:
			hipLaunchKernelGGL((k_pointwise_block_weight_layout<bf16_t>), grid, dim3(256), 0, st, static_cast<const bf16_t*>(w), static_cast<uint4*>(U), K, C, slabs,
					tiles);
			return 0;
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}

extern "C" int avhip_conv2d_pointwise_block(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias, const void *z,
		void *y, double alpha1, double alpha2, double beta, int activation)
{
	if (shape == nullptr || x == nullptr || U == nullptr || y == nullptr)
		return AVHIP_BAD_PARAM;
	if (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16)
		return AVHIP_UNSUPPORTED_DATATYPE;
	if (!block_shape_ok(*shape) || beta != 0.0 || (activation != ACT_LINEAR && activation != ACT_RELU))
		return AVHIP_NOT_SUPPORTED;
	hipStream_t st = static_cast<hipStream_t>(stream);
	return dtype == DT_FLOAT16 ? launch_block<f16_t>(st, *shape, x, U, bias, z, y, alpha1, alpha2, activation)
			: launch_block<bf16_t>(st, *shape, x, U, bias, z, y, alpha1, alpha2, activation);
}
