/*
 * conv_winograd_rows.hip -- 3x3 stride-1 convolution of 16-bit tensors by Winograd F(2,3) applied ALONG IMAGE ROWS ONLY,
 * in one kernel, for layers whose whole image (or a band of its rows) fits the LDS of a compute unit.
 *
 * Same formula as the other forward paths, y = act(alpha1 * conv(x, w) + bias + alpha2 * z) + beta * y
 * (include/Avocado/cuda_backend.h:822 of the reference; the reference's fused prototype is src/winograd_fused.cu:590-775,
 * launched at :789-805, and transforms in both directions).  Why one direction here: on the matrix cores of gfx950 a 16-bit
 * 3x3 layer is bound by the number of MFMA instructions, and what a two-dimensional transform saves there (2.25x) it gives
 * back in vector instructions, because its sixteen accumulator planes do not fit the register file and every finished plane
 * has to be folded into the outputs inside the k loop.  With the transform along one direction,
 *
 *     y[h, 2t + o] = sum_p A^T[o][p] * M_p[h, t],      M_p[h, t][k] = sum_{i, c} V_p[h + i, t][c] * U_p[i][k][c],
 *     V_p[r, t] = sum_j B^T[p][j] * x[r, 2t + j],      U_p[i]      = sum_j G[p][j] * w[k, i, j],
 *
 * the four planes M_0..M_3 of (output row, column pair) x filter stay in accumulator registers for the whole k loop
 * (k = 3 filter rows x C channels), the fold is four additions per pair of outputs, done once in the epilogue, and the matrix
 * cores issue 12 products per channel and pair of outputs instead of 18: two thirds of the direct kernel's MFMA work.
 * B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1], G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1], A^T = [1 1 1 0; 0 1 -1 -1]
 * (the one-dimensional factors of the F(2x2,3x3) tables of src/winograd_nonfused.cu:534-575, signs moved between B and A).
 *
 * Workgroup = 8 wavefronts = one tile of TH output rows x `pairs` column pairs of one image x 128 filters; GEMM rows are
 * (row, column pair), at most 128.  Wavefront (p, fh) owns plane M_p for 64 filters (32 of either 64-filter half of the block):
 * 4 x 2 MFMA tiles of 32 x 32, 128 accumulator registers.
 *   A operand: V_p lives in LDS, [phase slot][p][pixel = row * pairs + pair][128 bytes + 16], fp16; filter row i is a constant
 *              shift of i * pairs pixels, so a 32-row tile always reads 32 consecutive pixels (conflict-free).
 *              V is produced in the kernel, 32 channels per phase: every work-item loads the four pixels of one
 *              (row, pair, 8 channels), forms the four differences in packed fp16 (bf16 is converted first: exact within the
 *              fp16 range) and writes them; the next phase is transformed among the MFMAs of the current one.
 *   B operand: U_p[i] comes straight from global memory (L2) in MFMA register layout, written that way by the weight
 *              transform below: [phase][filter row][p][tile of 32 filters][16-channel slab][lane][16 bytes], one contiguous
 *              kilobyte per wavefront load, requested several slabs ahead through a ring of register sets.  No LDS, so no
 *              barrier inside a phase.
 *   Epilogue : runs inside the last phase.  That phase keeps its filters in registers and takes its products MFMA tile by MFMA
 *              tile (a unit); a finished unit's four planes go through one of two buffers in LDS, a work-item folds them into
 *              two output pixels x 4 filters, applies bias / residual / ReLU and stores 8 bytes per pixel (sixteen lanes: a whole
 *              128-byte line) while later units are multiplied: see the last phase in the kernel.
 *   Instances: per tensor type, channel count, activation (ReLU or none) and residual (present or not): nothing about the
 *              epilogue is decided by a branch inside the kernel.
 * All phases are written out (2, 4 or 8 for C = 64, 128, 256); V has four slots in LDS, a fifth phase takes the first slot again.
 * Limits: 16-bit tensors, 3x3, stride 1, dilation 1, zero padding value, C = 64, 128 or 256, K a multiple of 128, beta = 0,
 * LINEAR or RELU, images that tile into at most 128 (row, pair) positions per workgroup (see choose_tile), values within the
 * fp16 range.
 */
#include <atomic>

#include "conv_epilogue.hpp"
#include "mfma_core.hpp"

/* Instrumentation, compiled in with -DWINOGRAD_ROWS_STAMPS only: work-item 0 of every workgroup records the 100 MHz wall clock at
 * the phase boundaries of the kernel and avhip_debug_rows_stamps() copies the records of the last launch to the host. */
#ifdef WINOGRAD_ROWS_STAMPS
__device__ unsigned long long g_rows_stamps[4096 * 32];
#define STAMP(i) do { if (threadIdx.x == 0) g_rows_stamps[(blockIdx.x % 4096) * 32 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
extern "C" __attribute__((visibility("default"))) int avhip_debug_rows_stamps(void *out)
{
	return static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_rows_stamps), sizeof(g_rows_stamps)));
}
#else
#define STAMP(i) do { } while (0)
#endif

#ifndef ROWS_UNIT_VALU
#define ROWS_UNIT_VALU 10 /* vector-ALU instructions of the fold behind every MFMA of the last phase */
#endif
#ifndef ROWS_TRANSFORM_SLOTS
#define ROWS_TRANSFORM_SLOTS 1
#endif
#ifndef ROWS_STORE_POLICY
#define ROWS_STORE_POLICY 17 /* sc0 sc1: written through as the kernel runs, no streaming hint */
#endif

namespace
{
	using namespace avhip;

	constexpr int ROWS_MAX = 128; /* GEMM rows of a workgroup */
	constexpr int PIXELS_MAX = 136; /* pixels of one V plane: (TH + 2) * pairs */
	constexpr int POSITIONS = 4;
	constexpr int FILTER_ROWS = 3;
	constexpr int PHASE_CHANNELS = 32; /* channels transformed and multiplied per phase: two 16-channel MFMA slabs */
	constexpr int PHASE_SLABS = 2;
	constexpr int PITCH = 128 + 16; /* LDS bytes per pixel of a 64-channel slice */
	constexpr int POSITION_BYTES = (PIXELS_MAX + 1) * PITCH; /* one spare pixel behind every plane */
	constexpr int SLICE_BYTES = POSITIONS * POSITION_BYTES;
	constexpr int MAX_PHASES = 4;
	constexpr int V_SLACK = 8 * PITCH; /* what an MFMA row past the tile's last may read behind the last plane */
	constexpr int V_BYTES = (MAX_PHASES / 2) * SLICE_BYTES + V_SLACK;
	constexpr int ROWS_BLOCK_N = 128; /* filters per workgroup */
	constexpr int THREADS = 512;
	constexpr int OPERAND_BYTES = 1024; /* one MFMA operand of a wavefront: 64 lanes x 16 bytes */
	static_assert(V_BYTES <= 160 * 1024, "LDS of a compute unit");

	struct RowsGeom
	{
		int H, W, C, K, Ho, Wo, pad_h, pad_w;
		int TH; /* output rows of a tile */
		int pairs; /* column pairs of a tile: a tile is TH rows by 2 * pairs output pixels */
		unsigned int pairs_magic; /* 2^20 / pairs + 1: (v * magic) >> 20 == v / pairs for v < 1024 */
		int bands, segments; /* tiles down and across an image */
		int images;
		int filter_tiles; /* K / 32 */
	};

	/* Eight fp16 values as four packed pairs: arithmetic on a pair is one packed instruction */
	typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
	typedef float float2_t __attribute__((ext_vector_type(2)));
	struct Half8
	{
		half2_t h[4];
	};
	/* a - b on both halves with one instruction (the compiler takes a packed fp16 subtraction apart into two scalar ones and a
	 * pack; a packed add with the negate modifiers on its second operand is the same operation) */
	__device__ __forceinline__ half2_t pk_sub(half2_t a, half2_t b)
	{
		half2_t r;
		asm("v_pk_add_f16 %0, %1, %2 neg_lo:[0,1] neg_hi:[0,1]" : "=v"(r) : "v"(a), "v"(b));
		return r;
	}
	__device__ __forceinline__ Half8 to_half8(uint4 raw, f16_t)
	{
		return __builtin_bit_cast(Half8, raw);
	}
	/* bf16 -> fp16 through fp32, two values per conversion instruction (exact inside the fp16 range) */
	__device__ __forceinline__ Half8 to_half8(uint4 raw, bf16_t)
	{
		const unsigned int w[4] = { raw.x, raw.y, raw.z, raw.w };
		Half8 r;
#pragma unroll
		for (int i = 0; i < 4; i++)
		{
			const float2_t f = { __uint_as_float(w[i] << 16), __uint_as_float(w[i] & 0xFFFF0000u) };
			r.h[i] = __builtin_convertvector(f, half2_t);
		}
		return r;
	}

	/* U in MFMA operand layout.  One work-item = one lane's 16 bytes of (phase, filter row, tile of 32 filters, slab), all
	 * four positions. */
	template<typename TE>
	__global__ void k_rows_weight_transform(const TE *__restrict__ w, uint4 *__restrict__ U, int K, int C, int flip, int phases, int filter_tiles)
	{
		const int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
		const int64_t total = static_cast<int64_t>(phases) * FILTER_ROWS * filter_tiles * PHASE_SLABS * 64;
		if (e >= total)
			return;
		const int lane = static_cast<int>(e & 63);
		int64_t t = e >> 6;
		const int slab = static_cast<int>(t % PHASE_SLABS);
		t /= PHASE_SLABS;
		const int tile = static_cast<int>(t % filter_tiles);
		t /= filter_tiles;
		const int i = static_cast<int>(t % FILTER_ROWS);
		const int phase = static_cast<int>(t / FILTER_ROWS);
		const int k = tile * 32 + (lane & 31);
		const int c0 = phase * PHASE_CHANNELS + slab * 16 + (lane >> 5) * 8;
		float g[3][8];
#pragma unroll
		for (int j = 0; j < 3; j++)
		{
			const int wi = flip ? 2 - i : i, wj = flip ? 2 - j : j;
#pragma unroll
			for (int q = 0; q < 8; q++)
				g[j][q] = (k < K && c0 + q < C) ? Traits<TE>::load(w[((static_cast<int64_t>(k) * 3 + wi) * 3 + wj) * C + c0 + q]) : 0.0f;
		}
		union
		{
			uint4 u;
			_Float16 h[8];
		} out[POSITIONS];
#pragma unroll
		for (int q = 0; q < 8; q++)
		{
			out[0].h[q] = static_cast<_Float16>(g[0][q]);
			out[1].h[q] = static_cast<_Float16>(0.5f * (g[0][q] + g[1][q] + g[2][q]));
			out[2].h[q] = static_cast<_Float16>(0.5f * (g[0][q] - g[1][q] + g[2][q]));
			out[3].h[q] = static_cast<_Float16>(g[2][q]);
		}
#pragma unroll
		for (int p = 0; p < POSITIONS; p++)
			U[((((static_cast<int64_t>(phase) * FILTER_ROWS + i) * POSITIONS + p) * filter_tiles + tile) * PHASE_SLABS + slab) * 64 + lane] = out[p].u;
	}

	/* RELU, HAS_Z: the activation (ReLU or none) and whether a residual is added, fixed per instance: a branch on either inside the
	 * last phase would cut the scheduling regions in which a row tile's fold sits between the next one's MFMAs, and one copy of the
	 * last phase per combination behind a branch in front of it costs the register allocator its last registers. */
	template<typename TE, int PHASES, bool RELU, bool HAS_Z>
	__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_winograd_rows(const TE *__restrict__ x, const void *__restrict__ U,
			RowsGeom g, FloatEpilogue<TE> epi)
	{
		constexpr int STEPS = PHASES * FILTER_ROWS;
		constexpr unsigned int SZ = sizeof(TE);
		/* V of four phases (128 channels) fits LDS; layers with more channels reuse the slot of phase - 4.  Phase ph + 1 is written
		 * during the middle step of phase ph, by wavefronts that have passed the barrier of phase ph - 1, which nobody reaches
		 * before it is done with phase ph - 2: the slot's last readers (phase ph - 3) are long gone. */
		constexpr int RING = MAX_PHASES;
		__shared__ __attribute__((aligned(16))) char lds[V_BYTES];
		STAMP(0);
		epi.pin();
		keep_in_sgpr(g.pairs);
		keep_in_sgpr(g.TH);
		keep_in_sgpr(g.Ho);
		keep_in_sgpr(g.Wo);
		keep_in_sgpr(g.K);
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int p = wave & 3; /* plane of this wavefront */
		const int fh = wave >> 2; /* its 32 filters of either 64-filter half of the block */

		/* (image, band, segment) and filter block of workgroup number b.  Where workgroups share input (several tiles per image:
		 * neighbouring bands read two rows in common; several filter blocks: each reads the whole tile) they are renumbered so that the
		 * filter blocks of a tile and then the tiles of an image follow each other on one XCD, whose L2 then serves the second reader. */
		const unsigned int filter_blocks = static_cast<unsigned int>(g.filter_tiles) / 4u;
		const unsigned int all_blocks = static_cast<unsigned int>(g.images * g.bands * g.segments) * filter_blocks;
		auto tile_of = [&](unsigned int b, int &n, int &band, int &segment, int &kb) __attribute__((always_inline))
		{
			n = static_cast<int>(b);
			band = segment = kb = 0;
			if (g.bands * g.segments != 1 || filter_blocks != 1)
			{
				const unsigned int t = xcd_block(b, all_blocks);
				const unsigned int item = t / filter_blocks;
				kb = static_cast<int>(t - item * filter_blocks);
				const int per_image = g.bands * g.segments;
				n = static_cast<int>(item) / per_image;
				const int tile = static_cast<int>(item) - n * per_image;
				band = tile / g.segments;
				segment = tile - band * g.segments;
			}
		};
		/* transform side: this work-item's (row, pair, 8 channels) of every phase of a tile: where its four pixels are read and where
		 * its four planes go (what depends on the block is the same for all work-items and stays in scalar registers; a work-item
		 * adds its own constants) */
		auto pixels_of = [&](unsigned int b, unsigned int (&src)[4], int &dst) __attribute__((always_inline))
		{
			const int t_chunk = tid & 3;
			const int t_pixel = tid >> 2;
			const int t_row = static_cast<int>(__umul24(static_cast<unsigned int>(t_pixel), g.pairs_magic) >> 20);
			const int t_pair = t_pixel - t_row * g.pairs;
			const unsigned int t_base = (static_cast<unsigned int>(t_row * g.W + 2 * t_pair) * g.C + t_chunk * 8) * SZ;
			int n, band, segment, kb;
			tile_of(b, n, band, segment, kb);
			const int ih0 = band * g.TH + g.pad_h, v_rows = g.TH + 2;
			int top = -ih0 < 0 ? 0 : -ih0;
			top = top > v_rows ? v_rows : top;
			int bottom = ih0 + v_rows - g.H < 0 ? 0 : ih0 + v_rows - g.H;
			bottom = bottom > v_rows - top ? v_rows - top : bottom;
			const int real_rows = b < all_blocks ? v_rows - top - bottom : 0;
			const int iw0 = segment * 2 * g.pairs + g.pad_w; /* column of the tile's first pixel */
			const unsigned int origin = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(((n * g.H + ih0 + top) * g.W + iw0) * g.C * static_cast<int>(SZ)));
			const bool t_valid = t_row < real_rows;
#pragma unroll
			for (int j = 0; j < 4; j++)
			{
				const int iw = iw0 + 2 * t_pair + j;
				const bool inside = t_valid & (static_cast<unsigned int>(iw) < static_cast<unsigned int>(g.W));
				src[j] = inside ? origin + t_base + static_cast<unsigned int>(j * g.C) * SZ : OUT_OF_RANGE;
			}
			dst = (t_valid ? (top + t_row) * g.pairs + t_pair : PIXELS_MAX) * PITCH + t_chunk * 16;
		};
		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, static_cast<unsigned int>(g.images) * g.H * g.W * g.C * SZ);
		uint4 raw[4];
		auto load_x_from = [&](const unsigned int (&src)[4], int phase) __attribute__((always_inline))
		{
			/* (an out-of-range offset stays out of range with the phase added: tensors here are below 2 GiB) */
#pragma unroll
			for (int j = 0; j < 4; j++)
			{
				const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rx, static_cast<int>(src[j]), phase * PHASE_CHANNELS * static_cast<int>(SZ), 0);
				raw[j] = make_uint4(v[0], v[1], v[2], v[3]);
			}
		};
		/* (the ring of filter registers: see load_b) */
		constexpr int B_RING = FILTER_ROWS * PHASE_SLABS, B_AHEAD = B_RING - 1;
		Chunk bq[B_RING][2];
		const unsigned int block = blockIdx.y * gridDim.x + blockIdx.x;
		int n, band, segment, kb;
		tile_of(block, n, band, segment, kb);
		const int oh0 = band * g.TH;
		const int ow0 = segment * 2 * g.pairs;
		const int ih0 = oh0 + g.pad_h; /* input row of V row 0 */
		const int v_rows = g.TH + 2;
		int top = -ih0 < 0 ? 0 : -ih0; /* V rows above the image */
		top = top > v_rows ? v_rows : top;
		int bottom = ih0 + v_rows - g.H < 0 ? 0 : ih0 + v_rows - g.H; /* V rows below it */
		bottom = bottom > v_rows - top ? v_rows - top : bottom;
		const int real_rows = v_rows - top - bottom;

		/* B operand: this wavefront's two filter tiles are tiles fh and 2 + fh of the block's four (its 32 filters of either 64-filter half) */
		const unsigned int step_stride = static_cast<unsigned int>(POSITIONS * g.filter_tiles * PHASE_SLABS * OPERAND_BYTES);
		const __amdgpu_buffer_rsrc_t ru = make_buffer(U, static_cast<unsigned int>(STEPS) * step_stride);
		const unsigned int b_offset = static_cast<unsigned int>((p * g.filter_tiles + kb * 4 + fh) * PHASE_SLABS * OPERAND_BYTES + lane * 16);
		/* Filters go through a ring of register sets, one set = the two filter tiles of one 16-channel slab (two slabs per step),
		 * requested B_AHEAD slabs before they are multiplied: six sets, one phase's worth, which is what the last phase keeps in
		 * registers (rings of four and eight measured the same: the way ahead is not what the requests cost). */
		constexpr int SLABS_TOTAL = STEPS * PHASE_SLABS;
		auto load_b_at = [&](unsigned int offset, int slab, int tn, Chunk &into) __attribute__((always_inline)) /* slab: (step, slab of the step), over the whole k walk */
		{
			const int step = slab / PHASE_SLABS, sl = slab - step * PHASE_SLABS;
			const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(ru, static_cast<int>(offset + tn * 2 * PHASE_SLABS * OPERAND_BYTES),
					static_cast<int>(step * step_stride + sl * OPERAND_BYTES), 0);
			into.u = make_uint4(v[0], v[1], v[2], v[3]);
		};
		auto load_b_tile = [&](int slab, int tn, Chunk &into) __attribute__((always_inline))
		{
#ifdef ROWS_KNOCK_B /* timing experiment only: no filter requests inside the k loop (wrong results) */
			if (slab >= B_AHEAD)
				return;
#endif
			load_b_at(b_offset, slab, tn, into);
		};
		auto load_b = [&](int slab, Chunk (&set)[2]) __attribute__((always_inline))
		{
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
				load_b_tile(slab, tn, set[tn]);
		};

		unsigned int x_src[4];
		int v_dst;
		pixels_of(block, x_src, v_dst);
		auto load_x = [&](int phase) __attribute__((always_inline))
		{
#ifdef ROWS_KNOCK_X /* timing experiment only: no pixel requests inside the k loop (wrong results) */
			if (phase >= 2)
				return;
#endif
			load_x_from(x_src, phase);
		};
		/* B^T d for this work-item's pixels; work-items without a (row, pair) of the band write to a spare pixel, so that the
		 * transform is straight-line code the scheduler can spread among the MFMAs */
		auto transform = [&](int slot) __attribute__((always_inline))
		{
			Half8 d[4];
#pragma unroll
			for (int j = 0; j < 4; j++)
				d[j] = to_half8(raw[j], TE());
			Half8 v[POSITIONS];
#pragma unroll
			for (int q = 0; q < 4; q++)
			{
				v[0].h[q] = pk_sub(d[0].h[q], d[2].h[q]);
				v[1].h[q] = d[1].h[q] + d[2].h[q];
				v[2].h[q] = pk_sub(d[2].h[q], d[1].h[q]);
				v[3].h[q] = pk_sub(d[1].h[q], d[3].h[q]);
			}
			char *dst = lds + (slot >> 1) * SLICE_BYTES + (slot & 1) * 64 + v_dst;
#pragma unroll
			for (int q = 0; q < POSITIONS; q++)
				*reinterpret_cast<uint4*>(dst + q * POSITION_BYTES) = __builtin_bit_cast(uint4, v[q]);
		};
		/* the same in eight parts, one behind each pair of MFMAs of the step that carries it, ordered so that few converted pixels
		 * are alive at a time: d0, d2, plane 0, d1, plane 1, plane 2, d3, plane 3 */
		Half8 td[4];
		auto transform_part = [&](int slot, int part) __attribute__((always_inline))
		{
			constexpr int convert[8] = { 0, 2, -1, 1, -1, -1, 3, -1 }, plane[8] = { -1, -1, 0, -1, 1, 2, -1, 3 };
			if (convert[part] >= 0)
				td[convert[part]] = to_half8(raw[convert[part]], TE());
			else
			{
				const int q = plane[part];
				Half8 v;
#pragma unroll
				for (int e = 0; e < 4; e++)
					v.h[e] = q == 0 ? pk_sub(td[0].h[e], td[2].h[e]) : q == 1 ? td[1].h[e] + td[2].h[e] : q == 2 ? pk_sub(td[2].h[e], td[1].h[e]) : pk_sub(td[1].h[e], td[3].h[e]);
				char *dst = lds + (slot >> 1) * SLICE_BYTES + (slot & 1) * 64 + v_dst;
				*reinterpret_cast<uint4*>(dst + q * POSITION_BYTES) = __builtin_bit_cast(uint4, v);
			}
		};
		load_x(0); /* what the first MFMA waits for longest goes out first */
#pragma unroll
		for (int slab = 0; slab < B_AHEAD; slab++)
			load_b(slab, bq[slab]);

		/* V rows outside the image are zeros, in every plane and slice: the rows above the image are the first `top * pairs`
		 * pixels of a plane, the rows below it its last `bottom * pairs` */
		{
			const int above = top * g.pairs * 8, below = bottom * g.pairs * 8; /* 16-byte chunks per plane */
			const int skip = real_rows * g.pairs * 8;
			for (int plane = 0; plane < POSITIONS * ((PHASES < RING ? PHASES : RING) + 1) / 2; plane++)
				for (int e = tid; e < above + below; e += THREADS)
				{
					const int at = e < above ? e : e + skip;
					*reinterpret_cast<uint4*>(lds + plane * POSITION_BYTES + (at >> 3) * PITCH + (at & 7) * 16) = make_uint4(0u, 0u, 0u, 0u);
				}
		}

				const int kcol = kb * ROWS_BLOCK_N + (tid & 15) * 4; /* a work-item always stores the same 4 filters of each half of the block */

		/* MFMA operand address: lane l supplies GEMM row (l % 32) of a 32-row tile and the 8-channel half (l / 32) of a slab.  Rows
		 * past the tile's last read whatever follows in LDS (at most 127 + 2 * pairs pixels into a plane of 137: the next plane, or
		 * the slack behind the last one); their sums are never stored. */
		const int band_rows = g.TH * g.pairs;
		const int a_off = p * POSITION_BYTES + (lane & 31) * PITCH + (lane >> 5) * 16;
		const int tap_shift = g.pairs * PITCH;

		STAMP(1);
		transform(0);
		if (PHASES > 1)
			load_x(1);
		__syncthreads();
		STAMP(2);

		typename Mma<f16_t>::acc_t acc[4][2];
		/* A operands go through a ring of six register sets: the chunk four ahead of the one being multiplied is requested from LDS,
		 * chunk = (phase, filter row, slab, 32-row tile) in the order of use */
		constexpr int A_RING = 6, A_AHEAD = 4, STEP_CHUNKS_A = PHASE_SLABS * 4;
		Chunk a[A_RING];
		/* (slot: which of the ring's places in LDS holds the phase) */
		/* (With more phases than slots the addresses of phase ph + 4 are those of phase ph; left to itself the compiler keeps every
		 * sum of a base and an offset beyond the 16 bits of the instruction alive for four phases, some 26 registers at the peak.
		 * An opaque copy of the base per phase makes them things of one phase.) */
		int a_base[2] = { a_off, a_off };
		auto fresh_a_base = [&](int phase) __attribute__((always_inline))
		{
			if (PHASES > RING)
			{
				a_base[phase & 1] = a_off;
				asm volatile("" : "+v"(a_base[phase & 1]));
			}
		};
		auto read_a = [&](int phase, int i, int sl, int rt, Chunk &dst) __attribute__((always_inline))
		{
			const int slot = phase % RING;
			dst.u = *reinterpret_cast<const uint4*>(lds + (slot >> 1) * SLICE_BYTES + (slot & 1) * 64 + sl * 32 + i * tap_shift + rt * 32 * PITCH + a_base[phase & 1]);
		};
		/* All phases but the last, written out (the last one walks its products row tile by row tile, see below).  With more
		 * phases than LDS has slots a phase's V takes the slot of phase - RING, whose readers are long gone (above). */
		auto run_phases = [&]() __attribute__((always_inline))
		{
			constexpr int COUNT = PHASES - 1;
			constexpr int CHUNKS = COUNT * FILTER_ROWS * STEP_CHUNKS_A;
#pragma unroll
			for (int phase = 0; phase < COUNT; phase++)
			{
				fresh_a_base(phase + 1);
#pragma unroll
				for (int i = 0; i < FILTER_ROWS; i++)
				{
					const int step = phase * FILTER_ROWS + i;
					__builtin_amdgcn_sched_barrier(0); /* a step is one scheduling region, laid out by the groups at its end */
					/* The next phase's V, from pixels requested a phase ago, is formed among the MFMAs of the middle step and made
					 * visible by a barrier before the last one, so that the last step can read the first operands of the next phase
					 * ahead like any other: no phase starts with a barrier and a bare LDS latency. */
					const bool transform_here = i == 1;
					if (i == 2)
						__syncthreads();
#if ROWS_TRANSFORM_SLOTS
					if (transform_here)
					{
						/* The step that carries the transform is written slot by slot, a fence for the scheduler between slots: the
						 * requests of the slot, two MFMAs, one part of the transform.  (Laid out by groups like the other steps the
						 * scheduler put three quarters of the transform into one run of fifty vector instructions behind the fourth
						 * MFMA.) */
#pragma unroll
						for (int sl = 0; sl < PHASE_SLABS; sl++)
						{
							const int slab = step * PHASE_SLABS + sl;
#pragma unroll
							for (int rt = 0; rt < 4; rt++)
							{
								__builtin_amdgcn_sched_barrier(0);
								if (slab + B_AHEAD < SLABS_TOTAL && (rt == 0 || rt == 2))
									load_b_tile(slab + B_AHEAD, rt >> 1, bq[(slab + B_AHEAD) % B_RING][rt >> 1]);
								const int c = (step * PHASE_SLABS + sl) * 4 + rt;
								const int cn = c + A_AHEAD;
								if (cn < CHUNKS)
								{
									const int nstep = cn / STEP_CHUNKS_A, nphase = nstep / FILTER_ROWS;
									read_a(nphase, nstep % FILTER_ROWS, (cn / 4) % PHASE_SLABS, cn % 4, a[cn % A_RING]);
								}
#pragma unroll
								for (int tn = 0; tn < 2; tn++)
									Mma<f16_t>::run(bq[slab % B_RING][tn], a[c % A_RING], acc[rt][tn]);
								transform_part((phase + 1) % RING, sl * 4 + rt);
							}
						}
						__builtin_amdgcn_sched_barrier(0);
						if (phase + 2 < PHASES)
							load_x(phase + 2);
						continue;
					}
#endif
#pragma unroll
					for (int sl = 0; sl < PHASE_SLABS; sl++)
					{
						const int slab = step * PHASE_SLABS + sl; /* within the trip */
						if (slab + B_AHEAD < SLABS_TOTAL)
						{
							/* (a scalar offset is not part of a buffer's bounds check: slabs past the last ask for the last again) */
							const int ahead = slab + B_AHEAD;
							load_b(ahead, bq[(slab + B_AHEAD) % B_RING]);
						}
						if (transform_here && sl == 0)
							transform((phase + 1) % RING);
#pragma unroll
						for (int rt = 0; rt < 4; rt++)
						{
							const int c = (step * PHASE_SLABS + sl) * 4 + rt;
							const int cn = c + A_AHEAD; /* the chunk to request now */
							if (cn < CHUNKS)
							{
								const int nstep = cn / STEP_CHUNKS_A, nphase = nstep / FILTER_ROWS;
								read_a(nphase, nstep % FILTER_ROWS, (cn / 4) % PHASE_SLABS, cn % 4, a[cn % A_RING]);
							}
#pragma unroll
							for (int tn = 0; tn < 2; tn++)
							{
								/* filters as the rows of the MFMA tile, pixels as its columns: a lane then holds runs of four
								 * consecutive filters of one pixel, which the fold can move as 16-byte vectors */
								if (step == 0 && sl == 0)
									Mma<f16_t>::start(bq[slab % B_RING][tn], a[c % A_RING], acc[rt][tn]);
								else
									Mma<f16_t>::run(bq[slab % B_RING][tn], a[c % A_RING], acc[rt][tn]);
							}
						}
					}
					/* The order of the step's instructions: the filter requests of a slab go out in front of the slab's MFMAs and not a
					 * moment later (left to itself the scheduler sinks them to just before their use, to shorten the life of their
					 * registers); four vector instructions of the transform behind every MFMA issue while the matrix pipeline works,
					 * and a finished plane leaves for LDS at once. */
#pragma unroll
					for (int sl = 0; sl < PHASE_SLABS; sl++)
					{
						/* (the slab's two requests half a slab apart: 1 % better than back to back) */
						const bool requests = step * PHASE_SLABS + sl + B_AHEAD < SLABS_TOTAL;
						if (requests)
							__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
#pragma unroll
						for (int k = 0; k < 8; k++)
						{
							if (requests && k == 4)
								__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
							__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
							if (transform_here)
							{
								__builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
								if (k % 4 == 3)
									__builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
							}
						}
					}
					if (transform_here)
					{
						__builtin_amdgcn_sched_barrier(0);
						if (phase + 2 < PHASES)
						{
							const int next = phase + 2;
							load_x(next);
						}
					}
				}
			}
		};
		/* behind the first barrier: nothing could be read ahead */
#pragma unroll
		for (int c = 0; c < A_AHEAD; c++)
			read_a(0, 0, c / 4, c % 4, a[c]);
		/* A lane's accumulator registers 4i..4i+3 of tile (rt, tn) are filters tn * 64 + fh * 32 + 8i + 4 * (lane / 32) + 0..3 of GEMM row
		 * 32 rt + lane % 32. */
		typedef float quad_t __attribute__((ext_vector_type(4)));
		const __amdgpu_buffer_rsrc_t ry = make_buffer(epi.y + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K, static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ);
		const __amdgpu_buffer_rsrc_t rz = make_buffer(HAS_Z ? epi.z + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K : nullptr, HAS_Z ? static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ : 0u);
		constexpr std::integral_constant<bool, RELU> with_relu;
		constexpr std::integral_constant<bool, HAS_Z> with_z;
		{
			run_phases();
			/* The sums so far are pinned here: an MFMA has no side effect, so without a use in this block the chains of the row
			 * tiles that the last phase takes up later may be moved down to it, their pixel operands kept alive from every phase. */
#pragma unroll
			for (int rt = 0; rt < 4; rt++)
#pragma unroll
				for (int tn = 0; tn < 2; tn++)
					asm volatile("" : "+v"(acc[rt][tn]));
			/*
			 * The last phase, and the results out while it runs.  Its filters (six slabs, the whole ring) stay in registers and its
			 * products are taken unit by unit, a unit being one MFMA tile of sums: 32 GEMM rows (a row tile) by this wavefront's 32
			 * filters of one 64-filter half of the block.  A unit is final after an eighth of the phase; in the region after it goes
			 * into one of two fold buffers in the slice of LDS that the last phase does not read ([plane][32 rows][64 filters + 4]
			 * floats each), in the region after that its four sums per output are read back by the work-items that will fold them,
			 * and in the region after that it is folded and stored: a region holds the MFMAs of unit u, the four writes of unit
			 * u - 1, the four reads of unit u - 2 and the fold of unit u - 3, none of which waits for another or for a latency
			 * of LDS, and one barrier ends it: the writes are visible to the next region's reads, and the buffer that this
			 * region has read is free for the next region's writes.
			 */
			constexpr int LAST = PHASES - 1, LAST_SLAB = LAST * FILTER_ROWS * PHASE_SLABS;
			constexpr int UNIT_ROWS = 32, UNIT_FILTERS = ROWS_BLOCK_N / 2, UNIT_PITCH = UNIT_FILTERS + 4, UNIT_WORDS = POSITIONS * UNIT_ROWS * UNIT_PITCH;
			constexpr int ROW_TILE_CHUNKS = FILTER_ROWS * PHASE_SLABS, UNITS = 8;
			static_assert(B_RING == ROW_TILE_CHUNKS && A_RING == ROW_TILE_CHUNKS && 2 * UNIT_WORDS * 4 <= SLICE_BYTES,
					"one phase of filters and one row tile of pixels in the rings; both fold buffers in one slice");
			float *sm = reinterpret_cast<float*>(lds + ((LAST % RING) >> 1 == 0 ? SLICE_BYTES : 0));
			STAMP(5);
			load_b(LAST_SLAB + B_AHEAD, bq[(LAST_SLAB + B_AHEAD) % B_RING]);
			/* the six pixel operands of row tile 0; those of row tile rt + 1 take their places as the second unit of rt lets go of them */
#pragma unroll
			for (int c = 0; c < ROW_TILE_CHUNKS; c++)
				read_a(LAST, c / PHASE_SLABS, c % PHASE_SLABS, 0, a[c]);
			/* A work-item folds and stores, for one (row, pair) of a row tile, 4 filters of each half of the block: sixteen lanes
			 * read 64 consecutive words of a fold-buffer row (every bank once) and write one whole 128-byte line of y. */
			typename FloatEpilogue<TE>::template ColumnsT<4> columns[2];
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
				epi.request_columns(kcol + tn * UNIT_FILTERS, columns[tn]);
			unsigned int y_off[2][2];
			typedef unsigned int pair_t __attribute__((ext_vector_type(2)));
			pair_t residual[2][2][2]; /* [row tile parity][output pixel][half] */
			auto place = [&](int rt) __attribute__((always_inline)) /* where the two output pixels of this work-item's (row, pair) of row tile rt go */
			{
				/* (24-bit multiplies, which run at the full rate of the vector ALU, four times that of 32-bit ones: the launcher takes
				 * filter counts below 2^24 only, and an image of a tensor below 2 GiB has fewer than 2^24 pixels) */
				const unsigned int q = static_cast<unsigned int>(rt * UNIT_ROWS + (tid >> 4));
				const unsigned int r = __umul24(q, g.pairs_magic) >> 20;
				const int pair = static_cast<int>(q - __umul24(r, static_cast<unsigned int>(g.pairs)));
				const int oh = oh0 + static_cast<int>(r);
				const bool row_ok = (static_cast<int>(q) < band_rows) & (oh < g.Ho);
				const int ow = ow0 + 2 * pair;
				unsigned int first = (__umul24(__umul24(static_cast<unsigned int>(oh), static_cast<unsigned int>(g.Wo)) + static_cast<unsigned int>(ow), static_cast<unsigned int>(g.K)) + static_cast<unsigned int>(kcol)) * SZ;
				/* opaque: a select of a product invites a branch around the product, and a branch here ends the scheduling region */
				asm volatile("" : "+v"(first));
#pragma unroll
				for (int o = 0; o < 2; o++)
				{
					y_off[rt & 1][o] = (row_ok & (ow + o < g.Wo)) ? first + o * g.K * SZ : OUT_OF_RANGE;
					if constexpr (HAS_Z)
					{
#pragma unroll
						for (int tn = 0; tn < 2; tn++)
							residual[rt & 1][o][tn] = __builtin_bit_cast(pair_t, __builtin_amdgcn_raw_buffer_load_b64(rz, static_cast<int>(y_off[rt & 1][o]), tn * UNIT_FILTERS * SZ, 0));
					}
				}
			};
			auto hand_over = [&](int u) __attribute__((always_inline)) /* a finished unit into its fold buffer */
			{
				const int rt = u >> 1, tn = u & 1;
				float *dst = sm + tn * UNIT_WORDS + (p * UNIT_ROWS + (lane & 31)) * UNIT_PITCH + fh * 32 + (lane >> 5) * 4;
#pragma unroll
				for (int i = 0; i < 4; i++)
				{
					const typename Mma<f16_t>::acc_t &t = acc[rt][tn];
					const quad_t run = { t[4 * i], t[4 * i + 1], t[4 * i + 2], t[4 * i + 3] };
					*reinterpret_cast<quad_t*>(dst + i * 8) = run;
				}
			};
			quad_t held[2][POSITIONS]; /* a unit's four sums per output filter, read from its fold buffer a region before they are folded */
			auto fetch = [&](int u) __attribute__((always_inline))
			{
				const int tn = u & 1;
				const float *src = sm + tn * UNIT_WORDS + (tid >> 4) * UNIT_PITCH + (tid & 15) * 4;
#pragma unroll
				for (int q = 0; q < POSITIONS; q++)
					held[tn][q] = *reinterpret_cast<const quad_t*>(src + q * UNIT_ROWS * UNIT_PITCH);
			};
			auto fold_and_store = [&](int u) __attribute__((always_inline))
			{
				const int rt = u >> 1, tn = u & 1;
				const quad_t (&m)[POSITIONS] = held[tn];
				float out[2][4];
#pragma unroll
				for (int c = 0; c < 4; c++)
				{
					out[0][c] = m[0][c] + m[1][c] + m[2][c];
					out[1][c] = m[1][c] - m[2][c] - m[3][c];
				}
#pragma unroll
				for (int o = 0; o < 2; o++)
				{
					float t[4], zv[4];
					union
					{
						Pack<TE, 4> e;
						pair_t words;
					} cast;
					cast.words = residual[rt & 1][o][tn];
#pragma unroll
					for (int c = 0; c < 4; c++)
						zv[c] = HAS_Z ? Traits<TE>::load(cast.e.v[c]) : 0.0f;
					epi.template combine<RELU, HAS_Z, 4>(t, out[o], columns[tn], zv);
#pragma unroll
					for (int c = 0; c < 4; c++)
						cast.e.v[c] = Traits<TE>::store(t[c]);
					buffer_put<ROWS_STORE_POLICY>(ry, y_off[rt & 1][o] + tn * UNIT_FILTERS * SZ, cast.words);
				}
			};
			auto products = [&](int u) __attribute__((always_inline))
			{
				const int rt = u >> 1, tn = u & 1;
#pragma unroll
				for (int c = 0; c < ROW_TILE_CHUNKS; c++)
				{
					Mma<f16_t>::run(bq[(LAST_SLAB + c) % B_RING][tn], a[c], acc[rt][tn]);
					if (tn == 1 && rt < 3)
						read_a(LAST, c / PHASE_SLABS, c % PHASE_SLABS, rt + 1, a[c]);
				}
			};
#pragma unroll
			for (int u = 0; u < UNITS + 3; u++)
			{
				__builtin_amdgcn_sched_barrier(0);
#ifdef ROWS_KNOCK_LAST /* timing experiments only (wrong results): 1 no hand-over writes, 2 no fold, 8 no barriers */
				constexpr int knock = ROWS_KNOCK_LAST;
#else
				constexpr int knock = 0;
#endif
				if (u >= 3 && !(knock & 2))
					fold_and_store(u - 3);
				if (u >= 2 && u <= UNITS + 1 && !(knock & 2))
					fetch(u - 2);
				if (u >= 1 && u <= UNITS && !(knock & 1))
					hand_over(u - 1);
				if (u < UNITS)
				{
					/* (row tile rt is placed in the region of its second unit: its residual has two regions to arrive) */
					if ((u & 1) == 1)
						place(u >> 1);
					products(u);
					if (u >= 2)
						__builtin_amdgcn_sched_group_barrier(0x100, POSITIONS, 0); /* the reads of the fold buffer first */
#pragma unroll
					for (int c = 0; c < ROW_TILE_CHUNKS; c++)
					{
						__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
						if (u >= 1 && c < 4)
							__builtin_amdgcn_sched_group_barrier(0x200, 1, 0); /* (all four writes in front of the MFMAs measured 7 % slower over the phase) */
						if ((u & 1) == 1 && (u >> 1) < 3)
							__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
						__builtin_amdgcn_sched_group_barrier(0x002, ROWS_UNIT_VALU, 0);
					}
				}
				__builtin_amdgcn_sched_barrier(0);
				if (u == 1)
					STAMP(6);
				if (u == UNITS - 1)
					STAMP(7);
				STAMP(8 + u); /* (the end of every region of the last phase) */
				/* (behind region UNITS + 1 nothing is written any more: the last fetch and the last two folds need no barrier) */
				if (u <= UNITS && !(knock & 8))
					__syncthreads();
			}
			STAMP(3);
		}
		STAMP(4);
	}

	/* The tile (TH output rows by `pairs` column pairs) of a layer: what fits 128 GEMM rows, the V plane and one transform item per
	 * work-item and phase (rows of the tile's input inside the image x pairs <= 128), with the fewest tiles per image and, among
	 * those, the fewest halo rows.  th = 0 when nothing fits. */
	struct RowsTile
	{
		int th, pairs, bands, segments;
	};
	RowsTile choose_tile(const avhipConvShape &s)
	{
		RowsTile best = { 0, 0, 0, 0 };
		const int all_pairs = (s.Wo + 1) / 2;
		for (int pairs = 1; pairs <= all_pairs && pairs <= ROWS_MAX; pairs++)
		{
			const int segments = (all_pairs + pairs - 1) / pairs;
			if (pairs > 1 && (all_pairs + pairs - 2) / (pairs - 1) == segments)
				continue; /* a narrower tile gives the same number of segments: handled at that width, with more rows per tile */
			for (int th = s.Ho < ROWS_MAX ? s.Ho : ROWS_MAX; th >= 1; th--)
			{
				if (th * pairs > ROWS_MAX || (th + 2) * pairs > PIXELS_MAX)
					continue;
				bool fits = true;
				for (int oh0 = 0; oh0 < s.Ho && fits; oh0 += th)
				{
					const int first = oh0 + s.pad_h, last = first + th + 2; /* input rows [first, last) */
					const int lo = first < 0 ? 0 : first, hi = last > s.H ? s.H : last;
					if (hi > lo && (hi - lo) * pairs > ROWS_MAX)
						fits = false;
				}
				if (!fits)
					continue;
				const int bands = (s.Ho + th - 1) / th;
				if (best.th == 0 || bands * segments < best.bands * best.segments || (bands * segments == best.bands * best.segments && bands < best.bands))
					best = { th, pairs, bands, segments };
				break; /* smaller th only adds tiles */
			}
		}
		return best;
	}

	template<typename TE>
	int launch_rows(hipStream_t st, const avhipConvShape &s, const void *x, const void *U, const void *bias, const void *z, void *y, double alpha1,
			double alpha2, int activation)
	{
		if ((s.C != 64 && s.C != 128 && s.C != 256) || s.K % ROWS_BLOCK_N != 0 || s.K >= (1 << 24)) /* (24-bit products in the output offsets) */
			return AVHIP_NOT_SUPPORTED;
		if (!aligned_to(x, 16) || !aligned_to(U, 16) || !aligned_to(y, 16) || (z != nullptr && !aligned_to(z, 16)) || (bias != nullptr && !aligned_to(bias, 16)))
			return AVHIP_NOT_SUPPORTED;
		if (static_cast<int64_t>(s.N) * s.H * s.W * s.C * sizeof(TE) >= (1ll << 31) || static_cast<int64_t>(s.Ho) * s.Wo * s.K * sizeof(TE) >= (1ll << 31))
			return AVHIP_NOT_SUPPORTED;
		const RowsTile tile = choose_tile(s);
		if (tile.th == 0)
			return AVHIP_NOT_SUPPORTED;
		const int pairs = tile.pairs;
		RowsGeom g;
		g.TH = tile.th;
		g.H = s.H;
		g.W = s.W;
		g.C = s.C;
		g.K = s.K;
		g.Ho = s.Ho;
		g.Wo = s.Wo;
		g.pad_h = s.pad_h;
		g.pad_w = s.pad_w;
		g.pairs = pairs;
		g.pairs_magic = (1u << 20) / static_cast<unsigned int>(pairs) + 1u;
		g.bands = tile.bands;
		g.segments = tile.segments;
		g.images = s.N;
		g.filter_tiles = s.K / 32;
		const int64_t items = static_cast<int64_t>(s.N) * g.bands * g.segments;
		if (items >= (1ll << 31) || s.K / ROWS_BLOCK_N > 65535)
			return AVHIP_NOT_SUPPORTED;
		const FloatEpilogue<TE> epi { static_cast<const float*>(bias), static_cast<const TE*>(z), static_cast<TE*>(y), static_cast<float>(alpha1),
				static_cast<float>(alpha2), 0.0f, activation, s.K, true };
		const dim3 grid(static_cast<unsigned int>(items), static_cast<unsigned int>(s.K / ROWS_BLOCK_N));
		auto launch = [&](auto relu, auto residual)
		{
			constexpr bool R = decltype(relu)::value, Z = decltype(residual)::value;
			if (s.C == 256)
				hipLaunchKernelGGL((k_winograd_rows<TE, 8, R, Z>), grid, dim3(THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
			else if (s.C == 128)
				hipLaunchKernelGGL((k_winograd_rows<TE, 4, R, Z>), grid, dim3(THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
			else
				hipLaunchKernelGGL((k_winograd_rows<TE, 2, R, Z>), grid, dim3(THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
		};
		const bool relu = activation == ACT_RELU, residual = z != nullptr;
		if (relu && residual)
			launch(std::true_type(), std::true_type());
		else if (relu)
			launch(std::true_type(), std::false_type());
		else if (residual)
			launch(std::false_type(), std::true_type());
		else
			launch(std::false_type(), std::false_type());
		return 0;
	}
}

namespace
{
	std::atomic<int> rows_mode { 1 };
}
extern "C" int avhip_set_winograd_rows(int mode)
{
	return mode < 0 ? rows_mode.load() : rows_mode.exchange(mode);
}
extern "C" int avhip_conv2d_winograd_rows_plan(int dtype, const avhipConvShape *shape, int *workgroups, int *rows_used)
{
	if (shape == nullptr)
		return AVHIP_BAD_PARAM;
	const avhipConvShape &s = *shape;
	if (rows_mode.load() == 0 || (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16))
		return AVHIP_NOT_SUPPORTED;
	if (s.R != 3 || s.S != 3 || s.stride_h != 1 || s.stride_w != 1 || s.dil_h != 1 || s.dil_w != 1 || (s.C != 64 && s.C != 128 && s.C != 256)
			|| s.K % ROWS_BLOCK_N != 0 || s.N <= 0 || s.Ho <= 0 || s.Wo <= 0)
		return AVHIP_NOT_SUPPORTED;
	const RowsTile tile = choose_tile(s);
	if (tile.th == 0)
		return AVHIP_NOT_SUPPORTED;
	const int64_t groups = static_cast<int64_t>(s.N) * tile.bands * tile.segments * (s.K / ROWS_BLOCK_N);
	if (workgroups != nullptr)
		workgroups[0] = groups > 0x7FFFFFFF ? 0x7FFFFFFF : static_cast<int>(groups);
	if (rows_used != nullptr)
	{
		/* GEMM rows that are output pixel pairs, averaged over the tiles of an image (tiles at the right and lower edge are partial) */
		const int64_t useful = static_cast<int64_t>(s.Ho) * ((s.Wo + 1) / 2);
		rows_used[0] = static_cast<int>(useful / (tile.bands * tile.segments));
	}
	return 0;
}

extern "C" int64_t avhip_winograd_rows_weight_bytes(int K, int C)
{
	if (K <= 0 || C <= 0)
		return 0;
	const int64_t phases = (C + PHASE_CHANNELS - 1) / PHASE_CHANNELS, tiles = (K + 31) / 32;
	return phases * FILTER_ROWS * POSITIONS * tiles * PHASE_SLABS * OPERAND_BYTES;
}

extern "C" int avhip_winograd_rows_weight_transform(void *stream, int dtype, int invert, const void *w, void *U, int K, int C)
{
	if (w == nullptr || U == nullptr || K <= 0 || C <= 0)
		return AVHIP_BAD_PARAM;
	const int phases = (C + PHASE_CHANNELS - 1) / PHASE_CHANNELS, tiles = (K + 31) / 32;
	const int64_t total = static_cast<int64_t>(phases) * FILTER_ROWS * tiles * PHASE_SLABS * 64;
	const dim3 grid(ceil_div(total, 256));
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (dtype)
	{
		case DT_FLOAT16:
			hipLaunchKernelGGL((k_rows_weight_transform<f16_t>), grid, dim3(256), 0, st, static_cast<const f16_t*>(w), static_cast<uint4*>(U), K, C, invert, phases, tiles);
			return 0;
		case DT_BFLOAT16:
			hipLaunchKernelGGL((k_rows_weight_transform<bf16_t>), grid, dim3(256), 0, st, static_cast<const bf16_t*>(w), static_cast<uint4*>(U), K, C, invert, phases,
					tiles);
			return 0;
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}

extern "C" int avhip_conv2d_winograd_rows(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias, const void *z,
		void *y, double alpha1, double alpha2, double beta, int activation)
{
	if (shape == nullptr || x == nullptr || U == nullptr || y == nullptr)
		return AVHIP_BAD_PARAM;
	const avhipConvShape &s = *shape;
	if (s.N <= 0 || s.H <= 0 || s.W <= 0 || s.C <= 0 || s.K <= 0 || s.Ho <= 0 || s.Wo <= 0)
		return AVHIP_BAD_PARAM;
	if (s.R != 3 || s.S != 3 || s.stride_h != 1 || s.stride_w != 1 || s.dil_h != 1 || s.dil_w != 1 || beta != 0.0 || !is_simple_activation(activation))
		return AVHIP_NOT_SUPPORTED;
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (dtype)
	{
		case DT_FLOAT16:
			return launch_rows<f16_t>(st, s, x, U, bias, z, y, alpha1, alpha2, activation);
		case DT_BFLOAT16:
			return launch_rows<bf16_t>(st, s, x, U, bias, z, y, alpha1, alpha2, activation);
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}
