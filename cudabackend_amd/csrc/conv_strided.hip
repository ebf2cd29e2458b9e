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

	template<typename TE>
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
				const int r = static_cast<int>((static_cast<unsigned int>(pixel) * g.pw_magic) >> 20), c = pixel - r * g.PW;
				const int ih = ih0 + 2 * r + (plane >> 1), iw = iw0 + 2 * c + (plane & 1);
				const bool inside = (pixel < plane_pixels) & (static_cast<unsigned int>(ih) < static_cast<unsigned int>(g.H))
						& (static_cast<unsigned int>(iw) < static_cast<unsigned int>(g.W));
				x_src[k] = inside ? ((image + static_cast<unsigned int>(ih * g.W + iw)) * g.C + l_chunk * 8) * SZ : OUT_OF_RANGE;
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
		load_x(1, 0, raw); /* (a layer has at least two phases) */
		__syncthreads();
		SSTAMP(2);

		typename Mma<TE>::acc_t acc[S_ROW_TILES];
#pragma unroll
		for (int rt = 0; rt < S_ROW_TILES; rt++)
#pragma unroll
			for (int v = 0; v < 16; v++)
				acc[rt][v] = 0.0f;
		constexpr int A_RING = 6, A_AHEAD = 4;
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
		auto run_phase = [&](auto slot_tag, auto b_base_tag, int phase, int next) __attribute__((always_inline))
		{
			constexpr int SLOT = decltype(slot_tag)::value, B_BASE = decltype(b_base_tag)::value;
			constexpr int A_BASE = 0;
#pragma unroll
			for (int c = 0; c < A_AHEAD; c++)
				read_a(SLOT, c, a[(A_BASE + c) % A_RING]); /* behind the barrier of the phase: nothing could be read ahead */
#pragma unroll
			for (int tap = 0; tap < S_TAPS; tap++)
			{
				__builtin_amdgcn_sched_barrier(0);
				/* the next phase's planes: first half requested before this phase started, second half once the first is in LDS */
				if (tap == 3)
				{
					stash_x(SLOT ^ 1, 0, raw);
					__builtin_amdgcn_sched_barrier(0);
					load_x(next, 1, raw);
				}
				if (tap == 7)
					stash_x(SLOT ^ 1, 1, raw);
#pragma unroll
				for (int sl = 0; sl < S_SLABS; sl++)
				{
					const int slab = tap * S_SLABS + sl;
					load_b((phase * S_TAPS) * S_SLABS + slab + B_AHEAD, bq[(B_BASE + slab + B_AHEAD) % B_RING]);
#pragma unroll
					for (int rt = 0; rt < S_ROW_TILES; rt++)
					{
						const int c = slab * S_ROW_TILES + rt;
						if (c + A_AHEAD < PHASE_CHUNKS)
							read_a(SLOT, c + A_AHEAD, a[(A_BASE + c + A_AHEAD) % A_RING]);
						/* filters as the rows of the MFMA tile, pixels as its columns: a lane then holds runs of four consecutive filters
						 * of one pixel, which the hand-over can move as 16-byte vectors */
						Mma<TE>::run(bq[(B_BASE + slab) % B_RING], a[(A_BASE + c) % A_RING], acc[rt]);
					}
				}
#pragma unroll
				for (int sl = 0; sl < S_SLABS; sl++)
				{
					__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
#pragma unroll
					for (int k = 0; k < S_ROW_TILES; k++)
					{
						__builtin_amdgcn_sched_group_barrier(0x100, 1, 0); /* the LDS read four chunks ahead, in front of its MFMA */
						__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
						if ((tap == 3 || tap == 7) && sl == 0 && k % 2 == 1 && k / 2 < HALF)
							__builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
					}
				}
			}
			__builtin_amdgcn_sched_barrier(0);
		};
		/* trips of two phases (the channel count is a multiple of 64), one per half of LDS.  The planes of phase
		 * p + 1 are stored during phase p, into the half of LDS that phase p - 1 left at the barrier. */
		const int last = g.phases - 1;
		for (int phase = 0; phase < g.phases; phase += 2)
		{
			run_phase(std::integral_constant<int, 0>(), std::integral_constant<int, 0>(), phase, phase + 1);
			load_x(phase + 2 < last ? phase + 2 : last, 0, raw);
			__syncthreads();
			run_phase(std::integral_constant<int, 1>(), std::integral_constant<int, 0>(), phase + 1, phase + 2 < last ? phase + 2 : last);
			if (phase + 2 < g.phases)
			{
				load_x(phase + 3, 0, raw);
				__syncthreads();
			}
		}
		SSTAMP(3);

		/* hand-over and store: two passes of 128 GEMM rows; a work-item takes (row, 8 filters) eight times per pass */
		float *sm = reinterpret_cast<float*>(lds);
		const __amdgpu_buffer_rsrc_t ry = make_buffer(epi.y + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K, static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ);
		__amdgpu_buffer_rsrc_t rz = make_buffer(nullptr, 0);
		if (epi.z != nullptr)
			rz = make_buffer(epi.z + static_cast<int64_t>(n) * g.Ho * g.Wo * g.K, static_cast<unsigned int>(g.Ho * g.Wo * g.K) * SZ);
		const bool relu = epi.activation == ACT_RELU, has_z = epi.z != nullptr;
		const int kcol = kb * S_FILTERS + (tid & 31) * 8; /* a work-item always stores the same 8 filters */
		typename FloatEpilogue<TE>::template ColumnsT<8> columns;
		epi.request_columns(kcol, columns);
		constexpr int SWEEPS = S_FOLD_ROWS / (S_THREADS / 32); /* 8 */
#pragma unroll
		for (int pass = 0; pass < 2; pass++)
		{
			unsigned int y_off[SWEEPS];
			typename FloatEpilogue<TE>::template Residual<8> residual[SWEEPS];
#pragma unroll
			for (int it = 0; it < SWEEPS; it++)
			{
				const int q = pass * S_FOLD_ROWS + (tid >> 5) + it * (S_THREADS / 32);
				const int r = static_cast<int>((static_cast<unsigned int>(q) * g.pw_magic) >> 20), c = q - r * g.PW;
				const int oh = oh0 + r, ow = ow0 + c;
				const bool ok = (q < S_ROWS) & (r < g.TH) & (c < g.TW) & (oh < g.Ho) & (ow < g.Wo) & (kcol < g.K);
				y_off[it] = ok ? static_cast<unsigned int>((oh * g.Wo + ow) * g.K + kcol) * SZ : OUT_OF_RANGE;
				union
				{
					uint4 u;
					decltype(residual[0].raw) r8;
				} cast;
				cast.u = buffer_fetch<2>(rz, y_off[it]);
				residual[it].raw = cast.r8;
			}
			__syncthreads(); /* pass 0: everyone is done with the planes; pass 1: with the rows of pass 0 */
			/* A row of the buffer holds the 256 filters of a pixel as [first halves | second halves] of the 32 runs of 8 filters a
			 * work-item stores: run g, half h at word h * 128 + g * 4 (sixteen lanes reading one half of sixteen runs touch 64
			 * consecutive words).  This lane's accumulator registers 4i .. 4i + 3 of row tile rt are filters 32 * wave + 8i + 4 *
			 * (lane / 32) + 0..3 of pixel (lane % 32): run 4 * wave + i, half (lane / 32). */
			typedef float quad_t __attribute__((ext_vector_type(4)));
#pragma unroll
			for (int rt = 0; rt < 4; rt++)
			{
				if (pass * 4 + rt >= S_ROW_TILES)
					continue;
#pragma unroll
				for (int i = 0; i < 4; i++)
				{
					const typename Mma<TE>::acc_t &t = acc[pass * 4 + rt];
					const quad_t run = { t[4 * i], t[4 * i + 1], t[4 * i + 2], t[4 * i + 3] };
					*reinterpret_cast<quad_t*>(sm + (rt * 32 + (lane & 31)) * S_FOLD_PITCH + (lane >> 5) * 128 + (wave * 4 + i) * 4) = run;
				}
			}
			__syncthreads();
			auto leave = [&](auto with_relu, auto with_z) __attribute__((always_inline))
			{
#pragma unroll
				for (int it = 0; it < SWEEPS; it++)
				{
					const int row = (tid >> 5) + it * (S_THREADS / 32);
					const quad_t lo = *reinterpret_cast<const quad_t*>(sm + row * S_FOLD_PITCH + (tid & 31) * 4);
					const quad_t hi = *reinterpret_cast<const quad_t*>(sm + row * S_FOLD_PITCH + 128 + (tid & 31) * 4);
					const float v[8] = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
					const unsigned int offset = y_off[it];
					epi.template store_fast<decltype(with_relu)::value, decltype(with_z)::value, 8>(v, columns, residual[it], [&](auto words) __attribute__((always_inline))
					{
						buffer_put<17>(ry, offset, words); /* sc0 sc1: written through as the kernel runs */
					});
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
		}
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
		return s.R == 3 && s.S == 3 && s.stride_h == 2 && s.stride_w == 2 && s.dil_h == 1 && s.dil_w == 1 && s.C % 64 == 0 && s.C >= 64 && s.K % S_FILTERS == 0
				&& s.N > 0 && s.Ho > 0 && s.Wo > 0;
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
		hipLaunchKernelGGL((k_conv_strided<TE>), grid, dim3(S_THREADS), 0, st, static_cast<const TE*>(x), U, g, epi);
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
