/*
 * conv_strided.hip -- 3x3 stride-2 convolution of 16-bit tensors (the downsampling layers of a network) by implicit GEMM with the
 * input held in LDS as four parity planes and the filters fed to the matrix cores straight from L2.
 *
 * Same arithmetic as the implicit-GEMM forward of the reference (src/conv2d_implicit_gemm.cu:152-301, which is stride 1 only;
 * its entry point is cuda_convolution2dImplicitGemm, :303).  A general gather kernel re-reads every input pixel once per
 * filter tap that uses it and fetches the filters once per 128 output pixels; with stride 2 a tile of output pixels and its
 * input share no simple halo, which is why the image-tile kernel of the stride-1 layers does not apply.  Here
 *
 *   workgroup = 8 wavefronts = a tile of TH x TW output pixels of one image x 256 filters; GEMM rows are the tile's pixels at
 *               the pitch of a plane row (row q is pixel (q / PW, q % PW), PW = TW + 1), at most 224 = 7 MFMA tiles of 32;
 *   A operand : the input under the tile, (2 TH + 1) x (2 TW + 1) pixels, lies in LDS as four planes by the parity of its row
 *               and column relative to the tile's first input pixel: plane (pi, pj)[r][c] = x[ih0 + 2r + pi][iw0 + 2c + pj].  Tap
 *               (i, j) of output pixel (oh, ow) reads plane (i % 2, j % 2) at (oh + i / 2, ow + j / 2): for a GEMM row q that is
 *               plane pixel q + (i / 2) * PW + j / 2, a constant shift per tap, so a 32-row MFMA tile always reads 32 consecutive
 *               plane pixels (80-byte pitch: no bank conflicts).  32 channels per phase, two phases in LDS: the next phase is
 *               fetched and stored while the current one is multiplied, one barrier per phase;
 *   B operand : wavefront w owns filters 32w .. 32w + 31 for all rows (7 x 1 MFMA tiles, 112 accumulator registers); its
 *               operand comes from global memory (L2) in MFMA register layout, written that way once per weight tensor by
 *               avhip_conv2d_strided_weight_layout: [phase][tap][tile of 32 filters][slab][lane][16 bytes], one contiguous
 *               kilobyte per load, requested seven slabs ahead.  No LDS for the filters, no barrier inside a phase;
 *   every input pixel is read from memory once per workgroup (all 256 filters are here) and every filter once per tile.
 * Epilogue: the accumulators go through LDS in two passes so that a work-item stores 16 bytes of consecutive filters of one
 * pixel; bias / residual / ReLU as in the other kernels.
 * Limits: fp16 / bf16, 3x3, stride 2, dilation 1, zero padding value, C a multiple of 64, K a multiple of 256, beta = 0, LINEAR
 * or RELU, an output tile that fits (see choose_tile).
 */
#include <atomic>

#include "conv_epilogue.hpp"
#include "mfma_core.hpp"

#ifdef CONV_STRIDED_STAMPS
__device__ unsigned long long g_strided_stamps[4096 * 8];
#define SSTAMP(i) do { if (threadIdx.x == 0) g_strided_stamps[(blockIdx.x % 4096) * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
extern "C" __attribute__((visibility("default"))) int avhip_debug_strided_stamps(void *out)
{
	return static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_strided_stamps), sizeof(g_strided_stamps)));
}
#else
#define SSTAMP(i) do { } while (0)
#endif

namespace
{
	using namespace avhip;

	constexpr int S_THREADS = 512;
	constexpr int S_ROW_TILES = 7; /* MFMA tiles of 32 GEMM rows per workgroup */
	constexpr int S_ROWS = S_ROW_TILES * 32;
	constexpr int S_FILTERS = 256; /* per workgroup: 8 wavefronts x 32 */
	constexpr int S_TAPS = 9;
	constexpr int S_PHASE_CHANNELS = 32;
	constexpr int S_SLABS = 2; /* 16-channel MFMA slabs per phase */
	constexpr int S_PITCH = 64 + 16; /* LDS bytes per plane pixel of a phase */
	constexpr int S_PLANE_PIXELS = 256; /* allocated per plane: rows past the tile's last may read up to 223 + PW + 1 */
	constexpr int S_PLANE_BYTES = S_PLANE_PIXELS * S_PITCH;
	constexpr int S_PHASE_BYTES = 4 * S_PLANE_BYTES;
	constexpr int S_LDS = 2 * S_PHASE_BYTES; /* 163840: all of a compute unit */
	constexpr int S_LOADS = 4 * S_PLANE_PIXELS * (S_PHASE_CHANNELS * 2 / 16) / S_THREADS; /* 16-byte chunks per work-item and phase: 8 */
	constexpr int S_OPERAND = 1024;
	/* epilogue: [128 rows][256 filters + 4] floats per pass */
	constexpr int S_FOLD_ROWS = 128;
	constexpr int S_FOLD_PITCH = S_FILTERS + 4;
	static_assert(S_FOLD_ROWS * S_FOLD_PITCH * 4 <= S_LDS, "the hand-over reuses the LDS of the planes");
	static_assert(S_LDS <= 160 * 1024, "LDS of a compute unit");

	struct StridedGeom
	{
		int H, W, C, K, Ho, Wo, pad_h, pad_w;
		int TH, TW, PW; /* output tile, plane row pitch in pixels (TW + 1) */
		unsigned int pw_magic; /* 2^20 / PW + 1 */
		int tiles_h, tiles_w, images;
		int phases; /* C / 32 */
		int filter_tiles; /* K / 32 */
	};

	/* Weights in MFMA operand layout: one work-item = one lane's 16 bytes of (phase, tap, tile of 32 filters, slab). */
	template<typename TE>
	__global__ void k_strided_weight_layout(const TE *__restrict__ w, uint4 *__restrict__ U, int K, int C, int flip, int phases, int filter_tiles)
	{
		const int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
		const int64_t total = static_cast<int64_t>(phases) * S_TAPS * filter_tiles * S_SLABS * 64;
		if (e >= total)
			return;
		const int lane = static_cast<int>(e & 63);
		int64_t t = e >> 6;
		const int slab = static_cast<int>(t % S_SLABS);
		t /= S_SLABS;
		const int tile = static_cast<int>(t % filter_tiles);
		t /= filter_tiles;
		const int tap = static_cast<int>(t % S_TAPS);
		const int phase = static_cast<int>(t / S_TAPS);
		const int k = tile * 32 + (lane & 31);
		const int c0 = phase * S_PHASE_CHANNELS + slab * 16 + (lane >> 5) * 8;
		const int src_tap = flip ? S_TAPS - 1 - tap : tap;
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
					out.e[q] = w[(static_cast<int64_t>(k) * S_TAPS + src_tap) * C + c0 + q];
		}
		U[e] = out.u;
	}

	/* RELU, HAS_Z: the activation (ReLU or none) and whether a residual is added, fixed per instance: a branch on either in the tail
	 * would cut the scheduling regions in which the way out of a pair of row tiles sits between the MFMAs of the next pair. */
	template<typename TE, bool RELU, bool HAS_Z>
	__global__ __launch_bounds__(S_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_conv_strided(const TE *__restrict__ x, const void *__restrict__ U,
			StridedGeom g, FloatEpilogue<TE> epi)
	{
		constexpr unsigned int SZ = sizeof(TE);
		__shared__ __attribute__((aligned(16))) char lds[S_LDS];
		SSTAMP(0);
		epi.pin();
		keep_in_sgpr(g.PW);
		keep_in_sgpr(g.TH);
		keep_in_sgpr(g.TW);
		keep_in_sgpr(g.Ho);
		keep_in_sgpr(g.Wo);
		keep_in_sgpr(g.K);
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6; /* = this wavefront's tile of 32 filters */

		/* workgroups that share input (the filter blocks of a tile; neighbouring tiles of an image) follow each other on one XCD */
		int n = static_cast<int>(blockIdx.x), th = 0, tw = 0, kb = 0;
		if (g.tiles_h * g.tiles_w != 1 || gridDim.y != 1)
		{
			unsigned int item, filter_block;
			xcd_tile(item, filter_block);
			kb = static_cast<int>(filter_block);
			const int per_image = g.tiles_h * g.tiles_w;
			n = static_cast<int>(item) / per_image;
			const int tile = static_cast<int>(item) - n * per_image;
			th = tile / g.tiles_w;
			tw = tile - th * g.tiles_w;
		}
		const int oh0 = th * g.TH, ow0 = tw * g.TW;
		const int ih0 = 2 * oh0 + g.pad_h, iw0 = 2 * ow0 + g.pad_w;

		/* loader: work-item t fills 16-byte chunk (t % 4) of plane pixel slots t / 4 + 128 k, k < 8, of every phase: slot = plane *
		 * 256 + pixel; slots past a plane's (TH + 1) x PW pixels and pixels outside the image are zeros (out-of-range offsets) */
		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, static_cast<unsigned int>(g.images) * g.H * g.W * g.C * SZ);
		unsigned int x_src[S_LOADS];
		const int l_chunk = tid & 3;
		{
			const int plane_pixels = (g.TH + 1) * g.PW;
			const unsigned int image = static_cast<unsigned int>(n) * g.H * g.W;
#pragma unroll
			for (int k = 0; k < S_LOADS; k++)
			{
				const int slot = (tid >> 2) + k * (S_THREADS / 4);
				const int plane = slot >> 8, pixel = slot & (S_PLANE_PIXELS - 1);
				/* (24-bit multiplies, four times the rate of 32-bit ones: a tensor below 2 GiB of at least 64 channels has fewer than
				 * 2^24 pixels; what a pixel outside the image computes is not used) */
				const int r = static_cast<int>(__umul24(static_cast<unsigned int>(pixel), g.pw_magic) >> 20);
				const int c = pixel - static_cast<int>(__umul24(static_cast<unsigned int>(r), static_cast<unsigned int>(g.PW)));
				const int ih = ih0 + 2 * r + (plane >> 1), iw = iw0 + 2 * c + (plane & 1);
				const bool inside = (pixel < plane_pixels) & (static_cast<unsigned int>(ih) < static_cast<unsigned int>(g.H))
						& (static_cast<unsigned int>(iw) < static_cast<unsigned int>(g.W));
				const unsigned int at = image + __umul24(static_cast<unsigned int>(ih), static_cast<unsigned int>(g.W)) + static_cast<unsigned int>(iw);
				x_src[k] = inside ? (__umul24(at, static_cast<unsigned int>(g.C)) + l_chunk * 8) * SZ : OUT_OF_RANGE;
			}
		}
		/* LDS addresses are kept as a handful of base registers plus 16-bit immediates, and the bases are hidden from the optimiser:
		 * left to fold the constants it makes one address register per access beyond 64 KB and spills them */
		int l_base[2][2]; /* [half of LDS][loads 0-3 / 4-7] */
#pragma unroll
		for (int slot = 0; slot < 2; slot++)
#pragma unroll
			for (int upper = 0; upper < 2; upper++)
			{
				l_base[slot][upper] = slot * S_PHASE_BYTES + ((tid >> 2) + upper * 4 * (S_THREADS / 4)) * S_PITCH + l_chunk * 16;
				asm volatile("" : "+v"(l_base[slot][upper]));
			}
		/* a phase's planes come in two halves of four chunks per work-item, so that sixteen registers hold what is in flight */
		constexpr int HALF = S_LOADS / 2;
		uint4 raw[HALF];
		auto load_x = [&](int phase, int half, uint4 (&into)[HALF]) __attribute__((always_inline))
		{
#pragma unroll
			for (int k = 0; k < HALF; k++)
			{
				const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rx, static_cast<int>(x_src[half * HALF + k]), phase * S_PHASE_CHANNELS * static_cast<int>(SZ), 0);
				into[k] = make_uint4(v[0], v[1], v[2], v[3]);
			}
		};
		auto stash_x = [&](int slot, int half, const uint4 (&from)[HALF]) __attribute__((always_inline))
		{
#pragma unroll
			for (int k = 0; k < HALF; k++)
				*reinterpret_cast<uint4*>(lds + l_base[slot][half] + k * (S_THREADS / 4) * S_PITCH) = from[k];
		};
		/* Inside the k loop the next phase's planes come one chunk per tap, each stored two taps after it was requested (a ring of
		 * three register sets): vector-memory results return in order, so a filter request issued behind a plane request is usable
		 * only when that has landed, and four plane requests at once from all compute units queue up in HBM for longer than the
		 * filter ring looks ahead (phases 6.3 -> 5.9 us on 64 x 56 x 56 x 128 -> 256). */
		uint4 drip[3];
		auto request_chunk = [&](int phase, int k) __attribute__((always_inline)) /* chunk k of the phase's eight */
		{
			const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rx, static_cast<int>(x_src[k]), phase * S_PHASE_CHANNELS * static_cast<int>(SZ), 0);
			drip[k % 3] = make_uint4(v[0], v[1], v[2], v[3]);
		};
		auto store_chunk = [&](int slot, int k) __attribute__((always_inline))
		{
			*reinterpret_cast<uint4*>(lds + l_base[slot][k / HALF] + (k % HALF) * (S_THREADS / 4) * S_PITCH) = drip[k % 3];
		};
		uint4 raw_first[HALF]; /* (the second half of phase 0: only the prologue has the registers for both at once) */
		load_x(0, 0, raw);
		load_x(0, 1, raw_first);

		/* B operand: slab (phase, tap, slab of the phase) of this wavefront's filter tile is one contiguous kilobyte */
		const unsigned int tap_stride = static_cast<unsigned int>(g.filter_tiles * S_SLABS * S_OPERAND);
		const int slabs_total = g.phases * S_TAPS * S_SLABS;
		const __amdgpu_buffer_rsrc_t ru = make_buffer(U, static_cast<unsigned int>(g.phases * S_TAPS) * tap_stride);
		const unsigned int b_offset = static_cast<unsigned int>((kb * (S_FILTERS / 32) + wave) * S_SLABS * S_OPERAND + lane * 16);
		constexpr int B_RING = 6, B_AHEAD = 5; /* 18 slabs per phase: the ring stands at 0 when a phase starts */
		Chunk bq[B_RING];
		auto load_b = [&](int slab, Chunk &dst) __attribute__((always_inline)) /* slab over the whole k walk; past the last: the last again */
		{
			const int s = slab < slabs_total ? slab : slabs_total - 1;
			const int step = s / S_SLABS, sl = s - step * S_SLABS;
			const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(ru, static_cast<int>(b_offset), static_cast<int>(step * tap_stride + sl * S_OPERAND), 0);
			dst.u = make_uint4(v[0], v[1], v[2], v[3]);
		};
#pragma unroll
		for (int s = 0; s < B_AHEAD; s++)
			load_b(s, bq[s]);

		/* A operand address: lane l supplies GEMM row (l % 32) of a 32-row tile and the 8-channel half (l / 32) of a slab */
		int a_base[2][2][2]; /* [half of LDS][tap row i / 2][plane pair]: everything else of an operand's address is an immediate */
#pragma unroll
		for (int slot = 0; slot < 2; slot++)
#pragma unroll
			for (int down = 0; down < 2; down++)
#pragma unroll
				for (int pair = 0; pair < 2; pair++)
				{
					a_base[slot][down][pair] = slot * S_PHASE_BYTES + pair * 2 * S_PLANE_BYTES + down * g.PW * S_PITCH + (lane & 31) * S_PITCH + (lane >> 5) * 16;
					asm volatile("" : "+v"(a_base[slot][down][pair]));
				}
		SSTAMP(1);
		stash_x(0, 0, raw);
		stash_x(0, 1, raw_first);
		request_chunk(1, 0); /* (a layer has at least two phases) */
		request_chunk(1, 1);
		__syncthreads();
		SSTAMP(2);

		typename Mma<TE>::acc_t acc[S_ROW_TILES];
#pragma unroll
		for (int rt = 0; rt < S_ROW_TILES; rt++)
#pragma unroll
			for (int v = 0; v < 16; v++)
				acc[rt][v] = 0.0f;
		constexpr int A_RING = 6, A_AHEAD = 4;
		constexpr int HEAD_TAPS = 4, TAIL_TAPS = S_TAPS - HEAD_TAPS; /* of the last phase: taps walked slab by slab / row tile by row tile */
		constexpr int PHASE_CHUNKS = S_TAPS * S_SLABS * S_ROW_TILES; /* 126 A chunks per phase */
		static_assert(PHASE_CHUNKS % A_RING == 0 && (S_TAPS * S_SLABS) % B_RING == 0, "both operand rings stand at 0 when a phase starts");
		Chunk a[A_RING];
		/* chunk c of a phase = (tap, slab, row tile) in the order of use */
		auto read_a = [&](int slot, int c, Chunk &dst) __attribute__((always_inline))
		{
			const int tap = c / (S_SLABS * S_ROW_TILES), sl = (c / S_ROW_TILES) % S_SLABS, rt = c % S_ROW_TILES;
			const int i = tap / 3, j = tap % 3;
			const int plane = (i & 1) * 2 + (j & 1);
			dst.u = *reinterpret_cast<const uint4*>(lds + a_base[slot][i >> 1][plane >> 1] + (plane & 1) * S_PLANE_BYTES + (j >> 1) * S_PITCH + rt * 32 * S_PITCH + sl * 32);
		};
		/* One phase: 9 taps x 2 slabs x 7 MFMAs per wavefront.  SLOT: which half of LDS holds it; B_BASE: where the filter ring stands
		 * at its start. */
		auto run_phase = [&](auto slot_tag, auto last_tag, int phase, int next) __attribute__((always_inline))
		{
			const int after = next + 1 < g.phases ? next + 1 : next; /* (past the last phase: requested again, never stored) */
			/* LAST: the first HEAD_TAPS taps of the last phase only (no next phase to fetch; the remaining taps below) */
			constexpr int SLOT = decltype(slot_tag)::value, B_BASE = 0;
			constexpr bool LAST = decltype(last_tag)::value;
			constexpr int TAPS = LAST ? HEAD_TAPS : S_TAPS, CHUNKS = TAPS * S_SLABS * S_ROW_TILES;
			constexpr int A_BASE = 0;
#pragma unroll
			for (int c = 0; c < A_AHEAD; c++)
				read_a(SLOT, c, a[(A_BASE + c) % A_RING]); /* behind the barrier of the phase: nothing could be read ahead */
#pragma unroll
			for (int tap = 0; tap < TAPS; tap++)
			{
				__builtin_amdgcn_sched_barrier(0);
				/* the next phase's planes: chunk `tap` (requested two taps ago) into the other half of LDS, chunk tap + 2 requested;
				 * the last two taps request the first two chunks of the phase after that */
				if (!LAST && tap < S_LOADS)
					store_chunk(SLOT ^ 1, tap);
				const bool requests = !LAST && (tap + 2 < S_LOADS || tap + 2 - S_TAPS >= 0);
				if (!LAST && tap + 2 < S_LOADS)
					request_chunk(next, tap + 2);
				else if (!LAST && tap + 2 - S_TAPS >= 0)
					request_chunk(after, tap + 2 - S_TAPS);
#pragma unroll
				for (int sl = 0; sl < S_SLABS; sl++)
				{
					const int slab = tap * S_SLABS + sl;
					load_b((phase * S_TAPS) * S_SLABS + slab + B_AHEAD, bq[(B_BASE + slab + B_AHEAD) % B_RING]);
#pragma unroll
					for (int rt = 0; rt < S_ROW_TILES; rt++)
					{
						const int c = slab * S_ROW_TILES + rt;
						if (c + A_AHEAD < CHUNKS)
							read_a(SLOT, c + A_AHEAD, a[(A_BASE + c + A_AHEAD) % A_RING]);
						/* filters as the rows of the MFMA tile, pixels as its columns: a lane then holds runs of four consecutive filters
						 * of one pixel, which the hand-over can move as 16-byte vectors */
						Mma<TE>::run(bq[(B_BASE + slab) % B_RING], a[(A_BASE + c) % A_RING], acc[rt]);
					}
				}
#pragma unroll
				for (int sl = 0; sl < S_SLABS; sl++)
				{
					if (sl == 0 && requests)
						__builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
					else
						__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
#pragma unroll
					for (int k = 0; k < S_ROW_TILES; k++)
					{
						__builtin_amdgcn_sched_group_barrier(0x100, 1, 0); /* the LDS read four chunks ahead, in front of its MFMA */
						__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
						if (!LAST && tap < S_LOADS && sl == 0 && k == 1)
							__builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
					}
				}
			}
			__builtin_amdgcn_sched_barrier(0);
		};
		/* trips of two phases (the channel count is a multiple of 64), one per half of LDS.  The planes of phase
		 * p + 1 are stored during phase p, into the half of LDS that phase p - 1 left at the barrier. */
		int phase = 0;
		for (; phase + 2 < g.phases; phase += 2)
		{
			run_phase(std::integral_constant<int, 0>(), std::false_type(), phase, phase + 1);
			__syncthreads();
			run_phase(std::integral_constant<int, 1>(), std::false_type(), phase + 1, phase + 2);
			__syncthreads();
		}
		run_phase(std::integral_constant<int, 0>(), std::false_type(), phase, phase + 1);
		__syncthreads();
		SSTAMP(3);
		/*
		 * The last phase (in the second half of LDS; the first half is free from here on), and the results out while it runs.  Its
		 * first taps go slab by slab like any other phase.  The filters of the remaining taps are all held in registers and the
		 * products are taken two row tiles at a time, so that the sums of row tiles 0 and 1 are final when three more pairs are
		 * still to be multiplied: bias, residual, activation and rounding are applied in the layout of the accumulators (a lane
		 * holds runs of four consecutive filters of one pixel), the rounded runs pass through this wavefront's own piece of the
		 * free half of LDS (no barrier: LDS serves a wavefront's operations in order) and leave as 16-byte stores, four lanes per
		 * pixel, among the MFMAs of the next pair.  Only the last row tile's way out is left behind the loop.
		 */
		run_phase(std::integral_constant<int, 1>(), std::true_type(), phase + 1, phase + 1);
		constexpr int TAIL_SLABS = TAIL_TAPS * S_SLABS, HEAD_SLABS = HEAD_TAPS * S_SLABS;
		Chunk bl[TAIL_SLABS];
#pragma unroll
		for (int j = 0; j < TAIL_SLABS; j++)
		{
			if (j < B_AHEAD)
				bl[j] = bq[(HEAD_SLABS + j) % B_RING]; /* requested by the ring during the first taps */
			else
				load_b((phase + 1) * S_TAPS * S_SLABS + HEAD_SLABS + j, bl[j]);
		}
		const __amdgpu_buffer_rsrc_t ry = make_buffer(epi.y + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K, static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ);
		const __amdgpu_buffer_rsrc_t rz = make_buffer(HAS_Z ? epi.z + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K : nullptr, HAS_Z ? static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ : 0u);
		const int half = lane >> 5;
		const int kwave = kb * S_FILTERS + wave * 32; /* this wavefront's first filter */
		typedef float f32x4 __attribute__((ext_vector_type(4)));
		f32x4 bias[4]; /* of this lane's four filters in each of its four runs */
		{
			const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(epi.bias), 0, epi.bias != nullptr ? g.K * 4 : 0, 0x00020000);
#pragma unroll
			for (int i = 0; i < 4; i++)
				bias[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rb, (kwave + 8 * i + 4 * half) * 4, 0, 0));
		}
		constexpr int OUT_PITCH = 32 * static_cast<int>(SZ) + 16, OUT_BYTES = 64 * OUT_PITCH; /* [two row tiles of pixels][32 filters as stored] */
		static_assert((S_THREADS / 64) * OUT_BYTES <= S_PHASE_BYTES, "the wavefronts' pieces fit the free half of LDS");
		int out_put = wave * OUT_BYTES + (lane & 31) * OUT_PITCH + 4 * half * static_cast<int>(SZ);
		asm volatile("" : "+v"(out_put));
		int out_get = wave * OUT_BYTES + (lane >> 2) * OUT_PITCH + (lane & 3) * 16;
		asm volatile("" : "+v"(out_get));
		/* byte offset in y of GEMM row q of the tile (filter 0), or out of range (24-bit multiplies, which run at the full rate of the
		 * vector ALU: the launcher takes filter counts below 2^24 only, and an image of a tensor below 2 GiB has fewer than 2^24 pixels) */
		auto y_offset = [&](int q, int filter) __attribute__((always_inline))
		{
			const int r = static_cast<int>(__umul24(static_cast<unsigned int>(q), g.pw_magic) >> 20), c = q - static_cast<int>(__umul24(static_cast<unsigned int>(r), static_cast<unsigned int>(g.PW)));
			const int oh = oh0 + r, ow = ow0 + c;
			const bool ok = (r < g.TH) & (c < g.TW) & (oh < g.Ho) & (ow < g.Wo);
			/* (computed whether or not the pixel exists, and opaque: a select of a product invites a branch around the product, and a
			 * branch here ends the scheduling region) */
			unsigned int at = (__umul24(__umul24(static_cast<unsigned int>(oh), static_cast<unsigned int>(g.Wo)) + static_cast<unsigned int>(ow), static_cast<unsigned int>(g.K)) + static_cast<unsigned int>(filter)) * SZ;
			asm volatile("" : "+v"(at));
			return ok ? at : OUT_OF_RANGE;
		};
		/* The way out of a pair of row tiles (rt0, rt0 + 1) in thirteen parts, each of which sits behind one MFMA of the next pair:
		 * parts 0..7 round run i (of four) of row tile t (of two) in the layout of the accumulators and put it into the wavefront's
		 * piece of LDS; parts 8..12 read sixteen pixels each back as 16 bytes x 4 lanes per pixel and store them.  The residual of a pair
		 * is asked for a region ahead (fetch_z): runs (2 pair, 2 pair + 1) of the two lanes of a pixel are 32 consecutive bytes of
		 * z, 16 per lane, exchanged by the swap. */
		u32x4_t zraw[2][2];
		unsigned int zw[2][4];
		uint4 back[2];
		auto fetch_z = [&](int rt0, int count) __attribute__((always_inline))
		{
			if (HAS_Z)
			{
#pragma unroll
				for (int t = 0; t < count; t++)
#pragma unroll
					for (int pair = 0; pair < 2; pair++)
						zraw[t][pair] = __builtin_amdgcn_raw_buffer_load_b128(rz, static_cast<int>(y_offset((rt0 + t) * 32 + (lane & 31), kwave + 8 * (2 * pair + half))), 0, 2);
			}
		};
		auto way_out = [&](int rt0, int count, int part) __attribute__((always_inline))
		{
			if (part < 8)
			{
				const int t = part >> 2, i = part & 3, rt = rt0 + t;
				if (t >= count)
					return;
				if (HAS_Z && (i & 1) == 0)
				{
					const u32x4_t zr = zraw[t][i >> 1];
					const auto s0 = __builtin_amdgcn_permlane32_swap(zr[0], zr[2], false, false);
					const auto s1 = __builtin_amdgcn_permlane32_swap(zr[1], zr[3], false, false);
					zw[t][0] = s0[0]; /* run i, this lane's half */
					zw[t][1] = s1[0];
					zw[t][2] = s0[1]; /* run i + 1 */
					zw[t][3] = s1[1];
				}
				union
				{
					Pack<TE, 4> p;
					unsigned int w[2];
					uint2 u;
				} zin, out;
				zin.w[0] = HAS_Z ? zw[t][2 * (i & 1)] : 0u;
				zin.w[1] = HAS_Z ? zw[t][2 * (i & 1) + 1] : 0u;
#pragma unroll
				for (int e = 0; e < 4; e++)
				{
					float r = epi.alpha1 * acc[rt][4 * i + e] + bias[i][e];
					if (HAS_Z)
						r += epi.alpha2 * Traits<TE>::load(zin.p.v[e]);
					out.p.v[e] = Traits<TE>::store(RELU ? __builtin_fmaxf(r, 0.0f) : r);
				}
				*reinterpret_cast<uint2*>(lds + out_put + t * 32 * OUT_PITCH + 8 * i * static_cast<int>(SZ)) = out.u;
			}
			else
			{
				/* lane l: 16 bytes (l % 4) of pixel l / 4 + 16 it; read back a part ahead of its store */
				const int it = part - 8;
				if (it < 2 * count)
					back[it & 1] = *reinterpret_cast<const uint4*>(lds + out_get + it * 16 * OUT_PITCH);
				if (it >= 1 && it - 1 < 2 * count)
				{
					const uint4 run = back[(it - 1) & 1];
					const unsigned int offset = y_offset(rt0 * 32 + (it - 1) * 16 + (lane >> 2), kwave + (lane & 3) * 8);
					const u32x4_t words = { run.x, run.y, run.z, run.w };
					__builtin_amdgcn_raw_buffer_store_b128(words, ry, static_cast<int>(offset), 0, 17); /* sc0 sc1: written through as the kernel runs */
				}
			}
		};
		constexpr int WAY_OUT_PARTS = 13;
		/* chunk n of the tail = (pair of row tiles, tap, slab, row tile of the pair) in the order of use */
		auto tail_chunk = [&](int n, int &rt, int &tap, int &sl) __attribute__((always_inline))
		{
			constexpr int PER_PAIR = TAIL_SLABS * 2;
			const int pair = n / PER_PAIR < 3 ? n / PER_PAIR : 3; /* (the fourth "pair" is row tile 6 alone) */
			const int m = n - pair * PER_PAIR, width = pair < 3 ? 2 : 1;
			rt = pair * 2 + m % width;
			sl = (m / width) % S_SLABS;
			tap = HEAD_TAPS + m / (width * S_SLABS);
		};
		auto read_tail = [&](int n, Chunk &dst) __attribute__((always_inline))
		{
			int rt, tap, sl;
			tail_chunk(n, rt, tap, sl);
			const int i = tap / 3, j = tap % 3;
			const int plane = (i & 1) * 2 + (j & 1);
			dst.u = *reinterpret_cast<const uint4*>(lds + a_base[1][i >> 1][plane >> 1] + (plane & 1) * S_PLANE_BYTES + (j >> 1) * S_PITCH + rt * 32 * S_PITCH + sl * 32);
		};
		constexpr int TAIL_CHUNKS = TAIL_SLABS * S_ROW_TILES;
#pragma unroll
		for (int n = 0; n < A_AHEAD; n++)
			read_tail(n, a[n % A_RING]);
#pragma unroll
		for (int pair = 0; pair < 4; pair++)
		{
			/* The products of a pair of row tiles, slot by slot with a fence for the scheduler between slots: one MFMA and, behind it,
			 * the parts of the way out of the pair before that fall to the slot; the residual of this pair is asked for once those
			 * parts no longer need the one before. */
			const int width = pair < 3 ? 2 : 1, n0 = pair * TAIL_SLABS * 2, slots = TAIL_SLABS * width;
#pragma unroll
			for (int m = 0; m < slots; m++)
			{
				__builtin_amdgcn_sched_barrier(0);
				const int n = n0 + m;
				if (n + A_AHEAD < TAIL_CHUNKS)
					read_tail(n + A_AHEAD, a[(n + A_AHEAD) % A_RING]);
				int rt, tap, sl;
				tail_chunk(n, rt, tap, sl);
				Mma<TE>::run(bl[(tap - HEAD_TAPS) * S_SLABS + sl], a[n % A_RING], acc[rt]);
				if (pair > 0)
				{
					/* (in their order: a part that reads the piece of LDS back follows the parts that wrote what it reads) */
					const int first = slots >= WAY_OUT_PARTS ? (m < WAY_OUT_PARTS ? m : WAY_OUT_PARTS) : m * WAY_OUT_PARTS / slots;
					const int last = slots >= WAY_OUT_PARTS ? (m < WAY_OUT_PARTS ? m + 1 : WAY_OUT_PARTS) : (m + 1) * WAY_OUT_PARTS / slots;
#pragma unroll
					for (int part = first; part < last; part++)
						way_out(2 * (pair - 1), 2, part);
				}
				static_assert(TAIL_SLABS > 8, "the residual of a pair is asked for behind part 7 of the pair before");
				if (m == (pair > 0 ? 8 : 0))
					fetch_z(2 * pair, width);
			}
		}
		__builtin_amdgcn_sched_barrier(0);
#pragma unroll
		for (int part = 0; part < WAY_OUT_PARTS; part++)
			way_out(6, 1, part);
		SSTAMP(4);
	}

	/* The output tile of a layer: TH x TW with its rows at the plane pitch within 224 GEMM rows and its planes within the 256
	 * pixels allocated (the last rows read PW + 1 pixels past their own), the fewest tiles per image.  th = 0: nothing fits. */
	struct StridedTile
	{
		int th, tw, tiles_h, tiles_w;
	};
	StridedTile choose_strided_tile(const avhipConvShape &s)
	{
		StridedTile best = { 0, 0, 0, 0 };
		for (int tw = 1; tw <= s.Wo && tw <= 64; tw++)
		{
			const int pw = tw + 1;
			if (S_ROWS + pw + 1 > S_PLANE_PIXELS)
				break;
			for (int th = s.Ho; th >= 1; th--)
			{
				if ((th - 1) * pw + tw > S_ROWS || (th + 1) * pw > S_PLANE_PIXELS)
					continue;
				const int tiles_h = (s.Ho + th - 1) / th, tiles_w = (s.Wo + tw - 1) / tw;
				if (best.th == 0 || tiles_h * tiles_w < best.tiles_h * best.tiles_w)
					best = { th, tw, tiles_h, tiles_w };
				break;
			}
		}
		return best;
	}
	bool strided_shape_ok(const avhipConvShape &s)
	{
		return s.R == 3 && s.S == 3 && s.stride_h == 2 && s.stride_w == 2 && s.dil_h == 1 && s.dil_w == 1 && s.C % 64 == 0 && s.C >= 64 && s.C < (1 << 24) && s.K % S_FILTERS == 0
				&& s.N > 0 && s.Ho > 0 && s.Wo > 0 && s.K < (1 << 24); /* (24-bit products in the output offsets) */
	}
	std::atomic<int> strided_mode { 1 };

	template<typename TE>
	int launch_strided(hipStream_t st, const avhipConvShape &s, const void *x, const void *U, const void *bias, const void *z, void *y, double alpha1,
			double alpha2, int activation)
	{
		if (!aligned_to(x, 16) || !aligned_to(U, 16) || !aligned_to(y, 16) || (z != nullptr && !aligned_to(z, 16)) || (bias != nullptr && !aligned_to(bias, 16)))
			return AVHIP_NOT_SUPPORTED;
		if (static_cast<int64_t>(s.N) * s.H * s.W * s.C * sizeof(TE) >= (1ll << 31) || static_cast<int64_t>(s.Ho) * s.Wo * s.K * sizeof(TE) >= (1ll << 31)
				|| static_cast<int64_t>(s.C) * S_TAPS * s.K * sizeof(TE) >= (1ll << 31))
			return AVHIP_NOT_SUPPORTED;
		const StridedTile tile = choose_strided_tile(s);
		if (tile.th == 0)
			return AVHIP_NOT_SUPPORTED;
		StridedGeom g;
		g.H = s.H;
		g.W = s.W;
		g.C = s.C;
		g.K = s.K;
		g.Ho = s.Ho;
		g.Wo = s.Wo;
		g.pad_h = s.pad_h;
		g.pad_w = s.pad_w;
		g.TH = tile.th;
		g.TW = tile.tw;
		g.PW = tile.tw + 1;
		g.pw_magic = (1u << 20) / static_cast<unsigned int>(g.PW) + 1u;
		g.tiles_h = tile.tiles_h;
		g.tiles_w = tile.tiles_w;
		g.images = s.N;
		g.phases = s.C / S_PHASE_CHANNELS;
		g.filter_tiles = s.K / 32;
		const int64_t items = static_cast<int64_t>(s.N) * g.tiles_h * g.tiles_w;
		if (items >= (1ll << 31) || s.K / S_FILTERS > 65535)
			return AVHIP_NOT_SUPPORTED;
		const FloatEpilogue<TE> epi { static_cast<const float*>(bias), static_cast<const TE*>(z), static_cast<TE*>(y), static_cast<float>(alpha1),
				static_cast<float>(alpha2), 0.0f, activation, s.K, true };
		const dim3 grid(static_cast<unsigned int>(items), static_cast<unsigned int>(s.K / S_FILTERS));
		if (activation == ACT_RELU && z != nullptr)
			hipLaunchKernelGGL((k_conv_strided<TE, true, true>), grid, dim3(S_THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
		else if (activation == ACT_RELU)
			hipLaunchKernelGGL((k_conv_strided<TE, true, false>), grid, dim3(S_THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
		else if (z != nullptr)
			hipLaunchKernelGGL((k_conv_strided<TE, false, true>), grid, dim3(S_THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
		else
			hipLaunchKernelGGL((k_conv_strided<TE, false, false>), grid, dim3(S_THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
		return 0;
	}
}

extern "C" int avhip_set_conv_strided(int mode)
{
	return mode < 0 ? strided_mode.load() : strided_mode.exchange(mode);
}

extern "C" int avhip_conv2d_strided_plan(int dtype, const avhipConvShape *shape, int *workgroups, int *rows_used)
{
	if (shape == nullptr)
		return AVHIP_BAD_PARAM;
	const avhipConvShape &s = *shape;
	if (strided_mode.load() == 0 || (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16) || !strided_shape_ok(s))
		return AVHIP_NOT_SUPPORTED;
	const StridedTile tile = choose_strided_tile(s);
	if (tile.th == 0)
		return AVHIP_NOT_SUPPORTED;
	const int64_t groups = static_cast<int64_t>(s.N) * tile.tiles_h * tile.tiles_w * (s.K / S_FILTERS);
	if (workgroups != nullptr)
		workgroups[0] = groups > 0x7FFFFFFF ? 0x7FFFFFFF : static_cast<int>(groups);
	if (rows_used != nullptr)
		rows_used[0] = static_cast<int>(static_cast<int64_t>(s.Ho) * s.Wo / (tile.tiles_h * tile.tiles_w));
	return 0;
}

extern "C" int64_t avhip_conv2d_strided_weight_bytes(int K, int C)
{
	if (K <= 0 || C <= 0)
		return 0;
	const int64_t phases = (C + S_PHASE_CHANNELS - 1) / S_PHASE_CHANNELS, tiles = (K + 31) / 32;
	return phases * S_TAPS * tiles * S_SLABS * S_OPERAND;
}

extern "C" int avhip_conv2d_strided_weight_layout(void *stream, int dtype, int invert, const void *w, void *U, int K, int C)
{
	if (w == nullptr || U == nullptr || K <= 0 || C <= 0)
		return AVHIP_BAD_PARAM;
	const int phases = (C + S_PHASE_CHANNELS - 1) / S_PHASE_CHANNELS, tiles = (K + 31) / 32;
	const int64_t total = static_cast<int64_t>(phases) * S_TAPS * tiles * S_SLABS * 64;
	const dim3 grid(ceil_div(total, 256));
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (dtype)
	{
		case DT_FLOAT16:
			hipLaunchKernelGGL((k_strided_weight_layout<f16_t>), grid, dim3(256), 0, st, static_cast<const f16_t*>(w), static_cast<uint4*>(U), K, C, invert, phases,
					tiles);
			return 0;
		case DT_BFLOAT16:
			hipLaunchKernelGGL((k_strided_weight_layout<bf16_t>), grid, dim3(256), 0, st, static_cast<const bf16_t*>(w), static_cast<uint4*>(U), K, C, invert, phases,
					tiles);
			return 0;
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}

extern "C" int avhip_conv2d_strided(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias, const void *z, void *y,
		double alpha1, double alpha2, double beta, int activation)
{
	if (shape == nullptr || x == nullptr || U == nullptr || y == nullptr)
		return AVHIP_BAD_PARAM;
	const avhipConvShape &s = *shape;
	if (s.N <= 0 || s.H <= 0 || s.W <= 0 || s.C <= 0 || s.K <= 0 || s.Ho <= 0 || s.Wo <= 0)
		return AVHIP_BAD_PARAM;
	if (!strided_shape_ok(s) || beta != 0.0 || !is_simple_activation(activation))
		return AVHIP_NOT_SUPPORTED;
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (dtype)
	{
		case DT_FLOAT16:
			return launch_strided<f16_t>(st, s, x, U, bias, z, y, alpha1, alpha2, activation);
		case DT_BFLOAT16:
			return launch_strided<bf16_t>(st, s, x, U, bias, z, y, alpha1, alpha2, activation);
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}
