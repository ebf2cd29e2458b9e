/*
 * conv_thin.hip -- implicit-GEMM convolution for layers whose input has few channels and whose filter may be large: the
 * 7 x 7, stride-2 first layer of a residual network over three image planes is the type.
 *
 * Same arithmetic as the implicit-GEMM forward of the reference (src/conv2d_implicit_gemm.cu:152-301).  With so few
 * channels one tap holds a handful of bytes, so k is the flattened (tap, channel) index of a filter row, R * S * C elements
 * long, and a 16-byte MFMA operand chunk of an output pixel is put together from 16 / PB pieces of PB bytes, each from the
 * input pixel its tap reads (PB: the largest power of two that divides the bytes of a pixel, so a piece never straddles two
 * taps).  Gathering such pieces from global memory costs one cache-line look-up per work-item and piece; here the image
 * tile that a workgroup's 256 output pixels read is brought into LDS once, with neighbouring work-items reading neighbouring
 * addresses, and the pieces are gathered from LDS, which serves 32 scattered work-items per cycle.
 *
 * A work item is one tile of TH x TW = 256 output pixels of one image (TW a power of two, chosen per layer) times one block
 * of 64 filters; the resident workgroups (two per compute unit) walk the items in steps of the grid.  In LDS:
 *   the halo: the (TH-1)*stride + (R-1)*dilation + 1 image rows under the tile, zeros where the image ends;
 *   a table with, for every piece of k, its byte offset from the window origin of a pixel (the same for every pixel);
 *   the 64 filters of the current block, rows padded with zeros to whole 32-byte MFMA slabs (staged when the block changes,
 *   which for a workgroup is nearly never);
 *   the region through which the accumulators leave.
 * A wavefront owns 64 pixels (two MFMA tiles) by 64 filters; per 32-byte slab of k it gathers two operand chunks from the
 * halo, reads two filter chunks and issues four MFMAs.  No barrier inside the k loop.  The next item's halo is requested
 * before the accumulators leave and written once every wavefront is done with the current one.
 */
#include "conv_thin.hpp"
#include "mfma_core.hpp"
#include "persistent_gemm.hpp"
#include <algorithm>
#include <mutex>
#include <type_traits>
#include <vector>

/* Instrumentation, compiled in with -DCONV_THIN_STAMPS only: work-item 0 of every workgroup records the 100 MHz wall clock at
 * the phase boundaries of the kernel (start, first requests out, set-up done, and for its last item: first slab, last slab,
 * accumulators gone; next halo in LDS for the item before), and avhip_debug_thin_stamps() copies the records of the last
 * launch to the host. */
#ifdef CONV_THIN_STAMPS
__device__ unsigned long long g_thin_stamps[4096 * 8];
#define THIN_STAMP(i) do { if (threadIdx.x == 0) g_thin_stamps[(blockIdx.x % 4096) * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
extern "C" __attribute__((visibility("default"))) int avhip_debug_thin_stamps(void *out)
{
	return static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_thin_stamps), sizeof(g_thin_stamps)));
}
#else
#define THIN_STAMP(i) do { } while (0)
#endif

namespace
{
	using namespace avhip;

	constexpr int THIN_FILTERS = 64; /* filters per block */
	constexpr int THIN_LDS = 160 * 1024; /* most a workgroup may ask for: the LDS of a compute unit; it asks for what the layer needs (two fit up to 80 KB) */
	constexpr int THIN_MAX_K_BYTES = 1024;
	constexpr int THIN_MAX_PIXEL_BYTES = 64;
	constexpr unsigned int THIN_NO_PIECE = 0xFFFFFFFFu; /* table entry of a piece past the end of k */

	struct ThinGeom
	{
		int H, W, K, Ho, Wo, R, S;
		int pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, flip;
		int tw_shift; /* the tile is (256 >> tw_shift) rows of (1 << tw_shift) output pixels */
		unsigned int tiles_x, tiles_per_image, tiles, items; /* tiles: of all images; items: (filter block, tile) pairs */
		unsigned int pixel_bytes, k_bytes, kgroups; /* kgroups: 32-byte slabs of k, the last one padded */
		unsigned int halo_pitch, halo_pieces, pieces_per_row; /* halo row = pieces_per_row pieces = halo_pitch bytes, rows back to back */
		unsigned int step_rows, step_pieces; /* 256 pieces further on: this many rows and pieces down the halo */
		unsigned int halo_bytes, table_bytes; /* LDS regions, multiples of 16 */
		unsigned int w_pitch; /* LDS pitch of a padded filter row: an odd number of 16-byte units */
		unsigned int x_bytes, w_bytes;
		unsigned int filter_blocks;
		int narrow_rows; /* a tile's part of y spans less than 2 GiB: 32-bit offsets from its first pixel */
		int wide_halo; /* the halo is brought in as 16-byte pieces of image rows that start on 16-byte boundaries */
	};

	/* A piece of PB bytes: its register type, its load from a tensor (zeros at OUT_OF_RANGE) */
	template<int PB> struct ThinPiece;
	template<> struct ThinPiece<16>
	{
		typedef u32x4_t type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(off), 0, 0);
		}
	};
	template<> struct ThinPiece<8>
	{
		typedef u32x2_t type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b64(r, static_cast<int>(off), 0, 0);
		}
	};
	template<> struct ThinPiece<4>
	{
		typedef unsigned int type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b32(r, static_cast<int>(off), 0, 0);
		}
	};
	template<> struct ThinPiece<2>
	{
		typedef unsigned short type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b16(r, static_cast<int>(off), 0, 0);
		}
	};
	template<> struct ThinPiece<1>
	{
		typedef unsigned char type;
		__device__ static inline type get(__amdgpu_buffer_rsrc_t r, unsigned int off)
		{
			return __builtin_amdgcn_raw_buffer_load_b8(r, static_cast<int>(off), 0, 0);
		}
	};
	template<int PB>
	union ThinChunk
	{
		uint4 u;
		typename ThinPiece<PB>::type piece[16 / PB];
	};

	template<typename TE, int PB, typename Epi>
	__global__ __launch_bounds__(256, 2) void k_conv_thin(const TE *__restrict__ x, const TE *__restrict__ w, ThinGeom g, Epi epi)
	{
		epi.pin();
		constexpr int NP = 16 / PB;
		constexpr int W = Epi::wide;
		typedef typename ThinPiece<PB>::type piece_t;
		extern __shared__ __attribute__((aligned(16))) char lds[];
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int half = lane >> 5; /* which 16 bytes of a 32-byte slab this lane supplies */
		THIN_STAMP(0);

		unsigned int *table = reinterpret_cast<unsigned int*>(lds + g.halo_bytes);
		const unsigned int zero_at = g.halo_bytes + g.table_bytes; /* 16 bytes of zeros: what a piece past the end of k reads */
		char *filters = lds + zero_at + 16;
		char *drain = filters + THIN_FILTERS * g.w_pitch;
		const int TW = 1 << g.tw_shift;
		const __amdgpu_buffer_rsrc_t rx = make_buffer(x, g.x_bytes);
		const __amdgpu_buffer_rsrc_t rw = make_buffer(w, g.w_bytes);

		/* A workgroup walks the work items (filter block, image, tile) from its own number in steps of the grid: the filters stay
		 * in LDS while the filter block stays the same, which is nearly always. */
		struct Item
		{
			unsigned int fb, n;
			int oh0, ow0; /* first output pixel of the tile */
			int ih_base, column0; /* image row and byte column of the halo's first piece */
			unsigned int lead; /* bytes between the halo's first piece and its first pixel */
		};
		auto locate = [&](unsigned int item) __attribute__((always_inline))
		{
			Item it;
			it.fb = item / g.tiles;
			const unsigned int t = item - it.fb * g.tiles;
			it.n = t / g.tiles_per_image;
			const unsigned int in_image = t - it.n * g.tiles_per_image;
			const unsigned int tile_y = in_image / g.tiles_x, tile_x = in_image - tile_y * g.tiles_x;
			it.oh0 = static_cast<int>(tile_y) * (256 >> g.tw_shift);
			it.ow0 = static_cast<int>(tile_x) * TW;
			const int column_base = (it.ow0 * g.stride_w + g.pad_w) * static_cast<int>(g.pixel_bytes);
			it.lead = g.wide_halo ? static_cast<unsigned int>(column_base & 15) : 0u;
			it.column0 = column_base - static_cast<int>(it.lead);
			it.ih_base = it.oh0 * g.stride_h + g.pad_h;
			return it;
		};

		/* Filter rows f0 .. f0 + 63 lie back to back in w: read as aligned 16-byte chunks, written to the padded rows of LDS
		 * piece by piece (a chunk may run over the end of a filter row). */
		auto stage_filters = [&](int f0) __attribute__((always_inline))
		{
			const unsigned int total = static_cast<unsigned int>(g.K - f0 < THIN_FILTERS ? g.K - f0 : THIN_FILTERS) * g.k_bytes;
			const unsigned int w_first = static_cast<unsigned int>(f0) * g.k_bytes;
			const unsigned int tail_pieces = (g.kgroups * 32 - g.k_bytes) / PB;
			for (unsigned int idx = tid; idx < THIN_FILTERS * tail_pieces; idx += 256)
			{
				piece_t nothing = {};
				*reinterpret_cast<piece_t*>(filters + (idx & (THIN_FILTERS - 1)) * g.w_pitch + g.k_bytes + (idx / THIN_FILTERS) * PB) = nothing;
			}
			for (unsigned int off = tid * 16; off < total; off += 256 * 16)
			{
				ThinChunk<PB> chunk;
				chunk.u = buffer_fetch(rw, off + 16 <= total ? w_first + off : OUT_OF_RANGE);
				if (off + 16 > total) /* the one chunk that runs over the end of w */
				{
#pragma unroll
					for (int e = 0; e < NP; e++)
						chunk.piece[e] = ThinPiece<PB>::get(rw, off + e * PB < total ? w_first + off + e * PB : OUT_OF_RANGE);
				}
				unsigned int row = off / g.k_bytes, column = off - row * g.k_bytes;
#pragma unroll
				for (int e = 0; e < NP; e++)
				{
					if (off + e * PB < total)
						*reinterpret_cast<piece_t*>(filters + row * g.w_pitch + column) = chunk.piece[e];
					column += PB;
					if (column >= g.k_bytes)
					{
						column = 0;
						row++;
					}
				}
			}
		};

		/* The halo: the image rows under the tile, in pieces of SB bytes; consecutive work-items read consecutive pieces of a
		 * row.  SB = 16 where every image row starts on a 16-byte boundary: the halo then starts at the boundary at or before its
		 * first pixel (`lead` bytes earlier), and a piece lies inside an image row or outside as a whole.  The first pieces of a
		 * work-item are requested early (`request`) and written to LDS later (`commit`, which also moves the rest). */
		const unsigned int first_row = tid / g.pieces_per_row, first_piece = tid - first_row * g.pieces_per_row;
		const int row_bytes = g.W * static_cast<int>(g.pixel_bytes);
		struct Walk
		{
			unsigned int row, piece;
		};
		auto fetch_batch = [&](const Item &it, unsigned int first, Walk &at, auto &value) __attribute__((always_inline))
		{
			typedef typename std::remove_reference<decltype(value[0])>::type stage_t;
			constexpr int SB = sizeof(stage_t);
			constexpr int BATCH = sizeof(value) / SB;
#pragma unroll
			for (int u = 0; u < BATCH; u++)
			{
				const unsigned int q = first + u * 256 + tid;
				const int ih = it.ih_base + static_cast<int>(at.row);
				const int column = it.column0 + static_cast<int>(at.piece) * SB;
				const bool inside = (q < g.halo_pieces) & (ih >= 0) & (ih < g.H) & (column >= 0) & (column < row_bytes);
				value[u] = ThinPiece<SB>::get(rx, inside ? static_cast<unsigned int>((static_cast<int>(it.n) * g.H + ih) * row_bytes + column) : OUT_OF_RANGE);
				at.row += g.step_rows;
				at.piece += g.step_pieces;
				if (at.piece >= g.pieces_per_row)
				{
					at.piece -= g.pieces_per_row;
					at.row++;
				}
			}
		};
		auto store_batch = [&](unsigned int first, const auto &value) __attribute__((always_inline))
		{
			typedef typename std::remove_const<typename std::remove_reference<decltype(value[0])>::type>::type stage_t;
			constexpr int SB = sizeof(stage_t);
			constexpr int BATCH = sizeof(value) / SB;
#pragma unroll
			for (int u = 0; u < BATCH; u++)
			{
				const unsigned int q = first + u * 256 + tid;
				if (q < g.halo_pieces)
					*reinterpret_cast<stage_t*>(lds + q * SB) = value[u];
			}
		};
		constexpr int NARROW_BATCH = PB == 16 ? 4 : 8;
		u32x4_t wide_value[4];
		piece_t narrow_value[NARROW_BATCH];
		Walk walk;
		const bool wide = PB < 16 && g.wide_halo != 0;
		auto request = [&](const Item &it) __attribute__((always_inline))
		{
			walk.row = first_row;
			walk.piece = first_piece;
			if (wide)
				fetch_batch(it, 0u, walk, wide_value);
			else
				fetch_batch(it, 0u, walk, narrow_value);
		};
		auto commit = [&](const Item &it) __attribute__((always_inline))
		{
			if (wide)
			{
				store_batch(0u, wide_value);
				for (unsigned int first = 256 * 4; first < g.halo_pieces; first += 256 * 4)
				{
					fetch_batch(it, first, walk, wide_value);
					store_batch(first, wide_value);
				}
			}
			else
			{
				store_batch(0u, narrow_value);
				for (unsigned int first = 256 * NARROW_BATCH; first < g.halo_pieces; first += 256 * NARROW_BATCH)
				{
					fetch_batch(it, first, walk, narrow_value);
					store_batch(first, narrow_value);
				}
			}
		};

		unsigned int item = blockIdx.x;
		Item cur = locate(item);
		request(cur);
		THIN_STAMP(1);
		/* the table: entry (slab, half, piece) = offset of that piece of k from the window origin of a pixel */
		for (unsigned int idx = tid; idx < g.kgroups * 2 * NP; idx += 256)
		{
			const unsigned int b = (idx / NP) * 16 + (idx % NP) * PB;
			unsigned int rel = THIN_NO_PIECE;
			if (b < g.k_bytes)
			{
				const unsigned int tap = b / g.pixel_bytes, within = b - tap * g.pixel_bytes;
				int i = static_cast<int>(tap / g.S), j = static_cast<int>(tap - (tap / g.S) * g.S);
				if (g.flip)
				{
					i = g.R - 1 - i;
					j = g.S - 1 - j;
				}
				rel = static_cast<unsigned int>(i * g.dil_h) * g.halo_pitch + static_cast<unsigned int>(j * g.dil_w) * g.pixel_bytes + within;
			}
			table[idx] = rel;
		}
		if (tid < 4)
			reinterpret_cast<unsigned int*>(lds + zero_at)[tid] = 0u;
		stage_filters(static_cast<int>(cur.fb) * THIN_FILTERS);
		commit(cur);
		THIN_STAMP(2);
		__syncthreads();

		/* window origin of this lane's two output pixels (pixel m of the tile is row m >> tw_shift, column m & (TW - 1)) */
		unsigned int pixel_at[2];
#pragma unroll
		for (int tm = 0; tm < 2; tm++)
		{
			const int m = wave * 64 + tm * 32 + (lane & 31);
			pixel_at[tm] = static_cast<unsigned int>((m >> g.tw_shift) * g.stride_h) * g.halo_pitch
					+ static_cast<unsigned int>((m & (TW - 1)) * g.stride_w) * g.pixel_bytes;
		}
		const char *filter_row = filters + (lane & 31) * g.w_pitch + half * 16;
		const unsigned int *table_row = table + half * NP;

		for (;;)
		{
			THIN_STAMP(3);
			const int f0 = static_cast<int>(cur.fb) * THIN_FILTERS;
			const int kcol = f0 + drain_column<1, W>();
			typename Epi::template ColumnsT<W> columns;
			epi.load_columns(kcol, columns);
			const unsigned int origin[2] = { pixel_at[0] + cur.lead, pixel_at[1] + cur.lead };

			typename Mma<TE>::acc_t acc[2][2];
#pragma unroll
			for (int i = 0; i < 2; i++)
#pragma unroll
				for (int j = 0; j < 2; j++)
#pragma unroll
					for (int v = 0; v < 16; v++)
						acc[i][j][v] = 0;
			/* One slab: the table entries of the next slab are asked for before this slab's pieces (an LDS read that depends on
			 * an LDS read would otherwise pay the latency twice); only the last slab has pieces past the end of k (`checked`).
			 * Operands are not read a slab ahead: 2-byte pieces occupy a register each until they are packed, and two slabs of
			 * them in flight take more registers than two workgroups per compute unit leave; the other wavefronts hide the latency. */
			unsigned int rel[NP], rel_next[NP];
			auto entries = [&](unsigned int kg, unsigned int (&r)[NP]) __attribute__((always_inline))
			{
#pragma unroll
				for (int e = 0; e < NP; e++)
					r[e] = table_row[kg * 2 * NP + e];
			};
			auto slab = [&](unsigned int kg, auto checked) __attribute__((always_inline))
			{
				if (!decltype(checked)::value)
					entries(kg + 1, rel_next);
				Chunk a[2], b[2];
#pragma unroll
				for (int tm = 0; tm < 2; tm++)
				{
					ThinChunk<PB> chunk;
#pragma unroll
					for (int e = 0; e < NP; e++)
					{
						unsigned int at = origin[tm] + rel[e];
						if (decltype(checked)::value)
							at = rel[e] == THIN_NO_PIECE ? zero_at : at;
						chunk.piece[e] = *reinterpret_cast<const piece_t*>(lds + at);
					}
					a[tm].u = chunk.u;
				}
#pragma unroll
				for (int tn = 0; tn < 2; tn++)
					b[tn].u = *reinterpret_cast<const uint4*>(filter_row + tn * 32 * g.w_pitch + kg * 32);
#pragma unroll
				for (int tm = 0; tm < 2; tm++)
#pragma unroll
					for (int tn = 0; tn < 2; tn++)
						Mma<TE>::run(a[tm], b[tn], acc[tm][tn]);
#pragma unroll
				for (int e = 0; e < NP; e++)
					rel[e] = rel_next[e];
			};
			const unsigned int last = g.kgroups - 1;
			entries(0, rel);
			for (unsigned int kg = 0; kg < last; kg++)
				slab(kg, std::false_type());
			slab(last, std::true_type());
			THIN_STAMP(4);

			/* the next item's halo is asked for now and arrives while the accumulators leave */
			const unsigned int next_item = item + gridDim.x;
			const bool more = next_item < g.items;
			const Item next = locate(more ? next_item : item);
			if (more)
				request(next);

			const int oh0 = cur.oh0, ow0 = cur.ow0;
			const unsigned int n = cur.n;
			/* (the hand-over starts with a barrier: every wavefront is done with the halo and the filters) */
			bool gone = false;
			if constexpr (std::is_same<Epi, FloatEpilogue<TE>>::value && sizeof(TE) == 2)
			{
				/* the usual first layer (16-bit tensors, no residual, beta = 0): no branch in the epilogue, a buffer over the tile's
				 * part of y, rows outside the image at an out-of-range offset, runs written through as they go */
				if (epi.z == nullptr && epi.beta == 0.0f && g.narrow_rows)
				{
					constexpr unsigned int SZ = sizeof(TE);
					const __amdgpu_buffer_rsrc_t ry = make_buffer(epi.y + (static_cast<int64_t>(static_cast<int>(n) * g.Ho + oh0) * g.Wo + ow0) * g.K, 0x7FFFFFF0u);
					const int rows_left = g.Ho - oh0, columns_left = g.Wo - ow0;
					auto leave = [&](auto relu) __attribute__((always_inline))
					{
						drain_tile_private<TE, 2, W>(drain, acc, [&](int row, const float (&v)[W], int) __attribute__((always_inline))
						{
							const int ty = row >> g.tw_shift, tx = row & (TW - 1);
							const unsigned int offset = (ty < rows_left && tx < columns_left && kcol < g.K) ?
									static_cast<unsigned int>((ty * g.Wo + tx) * g.K + kcol) * SZ : OUT_OF_RANGE;
							typename Epi::template Residual<W> none;
							epi.template store_fast<decltype(relu)::value, false, W>(v, columns, none, [&](auto words) __attribute__((always_inline))
							{
								buffer_put<STORE_STREAM_THROUGH>(ry, offset, words);
							});
						});
					};
					if (epi.activation == ACT_RELU)
						leave(std::true_type());
					else
						leave(std::false_type());
					gone = true;
				}
			}
			if (!gone)
				drain_tile_private<TE, 2, W>(drain, acc, [&](int row, const typename Epi::scalar_t (&v)[W], int) __attribute__((always_inline))
			{
				const int oh = oh0 + (row >> g.tw_shift), ow = ow0 + (row & (TW - 1));
				if (oh < g.Ho && ow < g.Wo && kcol < g.K)
					epi.template store_at<ACT_SIMPLE, true, W>((static_cast<int64_t>(static_cast<int>(n) * g.Ho + oh) * g.Wo + ow) * g.K + kcol, kcol, v, columns,
							nullptr);
			});
			THIN_STAMP(5);
			if (!more)
				break;
			commit(next);
			if (next.fb != cur.fb)
				stage_filters(static_cast<int>(next.fb) * THIN_FILTERS);
			THIN_STAMP(6);
			__syncthreads();
			cur = next;
			item = next_item;
		}
	}

	/* a workgroup stores 64 filters of a pixel: int8 results are half a cache line, which is best written through */
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
	unsigned int round_up(unsigned int v, unsigned int to)
	{
		return (v + to - 1) / to * to;
	}
}

namespace
{
	/* Whether `kernel` may be launched with up to THIN_LDS bytes of dynamic LDS on the current device: asked of the runtime once
	 * per kernel instance and device, remembered afterwards. */
	bool large_lds_allowed(const void *kernel)
	{
		struct Answer
		{
			const void *kernel;
			int device;
			bool allowed;
		};
		static std::mutex mutex;
		static std::vector<Answer> answers;
		int device = 0;
		if (hipGetDevice(&device) != hipSuccess)
		{
			(void) hipGetLastError();
			return false;
		}
		std::lock_guard<std::mutex> lock(mutex);
		for (const Answer &a : answers)
			if (a.kernel == kernel && a.device == device)
				return a.allowed;
		const bool allowed = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, THIN_LDS) == hipSuccess;
		if (!allowed)
			(void) hipGetLastError();
		answers.push_back({ kernel, device, allowed });
		return allowed;
	}
}

namespace avhip
{
	template<typename TE, typename Epi>
	bool conv_thin_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &caller_epi)
	{
		const Epi epi = for_partial_lines(caller_epi);
		const int pixel_bytes = s.C * static_cast<int>(sizeof(TE));
		const int64_t k_bytes = static_cast<int64_t>(s.R) * s.S * pixel_bytes;
		if (pixel_bytes > THIN_MAX_PIXEL_BYTES || k_bytes > THIN_MAX_K_BYTES)
			return false;
		int pb = 16;
		while (pb > 1 && (pixel_bytes % pb != 0 || !aligned_to(x, pb)))
			pb /= 2;
		if (pb < static_cast<int>(sizeof(TE)) || !aligned_to(w, 16))
			return false;
		/* whole runs of Epi::wide filters leave with one vector store */
		if (!epi.vec || s.K % Epi::wide != 0 || !aligned_to(epi.y, 16) || (epi.z != nullptr && !aligned_to(epi.z, 16)))
			return false;
		const int64_t x_bytes = static_cast<int64_t>(s.N) * s.H * s.W * pixel_bytes, w_bytes = static_cast<int64_t>(s.K) * k_bytes;
		if (x_bytes >= (1ll << 31) || w_bytes >= (1ll << 31))
			return false;

		ThinGeom g;
		g.kgroups = static_cast<unsigned int>((k_bytes + 31) / 32);
		g.w_pitch = g.kgroups * 32 + 16;
		g.table_bytes = round_up(g.kgroups * 2 * (16 / pb) * 4, 16);
		const unsigned int drain_bytes = 4 * PrivateDrainRows<2, Epi::wide>::bytes;
		const unsigned int fixed_bytes = g.table_bytes + 16 + THIN_FILTERS * g.w_pitch + drain_bytes;
		/* image rows that start on 16-byte boundaries are brought in as 16-byte pieces, from the boundary at or before the first
		 * pixel of the halo: up to 16 - pb bytes more per row */
		g.wide_halo = (pb < 16 && (static_cast<int64_t>(s.W) * pixel_bytes) % 16 == 0 && aligned_to(x, 16)) ? 1 : 0;
		const int stage_bytes = g.wide_halo ? 16 : pb;
		auto halo_of = [&](int shift, unsigned int &rows, unsigned int &pitch)
		{
			const int tw = 1 << shift, th = 256 >> shift;
			const int64_t r = static_cast<int64_t>(th - 1) * s.stride_h + static_cast<int64_t>(s.R - 1) * s.dil_h + 1;
			const int64_t c = static_cast<int64_t>(tw - 1) * s.stride_w + static_cast<int64_t>(s.S - 1) * s.dil_w + 1;
			const int64_t p = g.wide_halo ? (c * pixel_bytes + 16 - pb + 15) / 16 * 16 : c * pixel_bytes;
			rows = static_cast<unsigned int>(std::min<int64_t>(r, 1 << 20));
			pitch = static_cast<unsigned int>(std::min<int64_t>(p, 1 << 20));
			return r * p;
		};
		/* the tile shape: as few tiles as possible, then the smallest halo */
		int best_shift = -1;
		int64_t best_tiles = 0, best_halo = 0;
		for (int shift = 0; shift <= 8; shift++)
		{
			const int tw = 1 << shift, th = 256 >> shift;
			unsigned int rows, pitch;
			const int64_t halo = halo_of(shift, rows, pitch);
			if (halo + 16 + fixed_bytes > THIN_LDS)
				continue;
			const int64_t tiles = static_cast<int64_t>((s.Ho + th - 1) / th) * ((s.Wo + tw - 1) / tw);
			if (best_shift < 0 || tiles < best_tiles || (tiles == best_tiles && halo < best_halo))
			{
				best_shift = shift;
				best_tiles = tiles;
				best_halo = halo;
			}
		}
		if (best_shift < 0)
			return false;
		/* images much smaller than a tile leave most of the MFMA rows empty */
		if (static_cast<int64_t>(s.Ho) * s.Wo * 10 < best_tiles * 256 * 3)
			return false;
		if (best_tiles * s.N * ((s.K + THIN_FILTERS - 1) / THIN_FILTERS) >= (1ll << 31))
			return false;
		const int tw = 1 << best_shift;
		g.H = s.H;
		g.W = s.W;
		g.K = s.K;
		g.Ho = s.Ho;
		g.Wo = s.Wo;
		g.R = s.R;
		g.S = s.S;
		g.pad_h = s.pad_h;
		g.pad_w = s.pad_w;
		g.stride_h = s.stride_h;
		g.stride_w = s.stride_w;
		g.dil_h = s.dil_h;
		g.dil_w = s.dil_w;
		g.flip = s.mode != 0 ? 1 : 0;
		g.tw_shift = best_shift;
		g.tiles_x = static_cast<unsigned int>((s.Wo + tw - 1) / tw);
		g.tiles_per_image = static_cast<unsigned int>(best_tiles);
		g.pixel_bytes = static_cast<unsigned int>(pixel_bytes);
		g.k_bytes = static_cast<unsigned int>(k_bytes);
		unsigned int halo_rows;
		halo_of(best_shift, halo_rows, g.halo_pitch);
		g.pieces_per_row = g.halo_pitch / stage_bytes;
		g.halo_pieces = halo_rows * g.pieces_per_row;
		g.step_rows = 256 / g.pieces_per_row;
		g.step_pieces = 256 % g.pieces_per_row;
		g.halo_bytes = round_up(halo_rows * g.halo_pitch, 16);
		g.x_bytes = static_cast<unsigned int>(x_bytes);
		g.w_bytes = static_cast<unsigned int>(w_bytes);
		g.filter_blocks = static_cast<unsigned int>((s.K + THIN_FILTERS - 1) / THIN_FILTERS);
		g.narrow_rows = (256ll * s.Wo * s.K * static_cast<int64_t>(sizeof(TE)) < (1ll << 31)) ? 1 : 0;
		g.tiles = static_cast<unsigned int>(best_tiles * s.N);
		g.items = g.tiles * g.filter_blocks;
		const unsigned int lds_bytes = g.halo_bytes + fixed_bytes;
		/* the workgroups that stay resident (two per compute unit by their registers, one where LDS allows no more) share the
		 * work items */
		const unsigned int resident = persistent_workgroups(1 << 30) / (lds_bytes > 80u * 1024u ? 2 : 1);
		const dim3 grid(std::min(g.items, resident));
		/* more than 64 KB of dynamic LDS needs the kernel's say-so, given once per instance and device; where that fails nothing
		 * is launched and the caller's other kernels take the layer */
#define AVHIP_THIN(PB) \
		if (lds_bytes > 64u * 1024u && !large_lds_allowed(reinterpret_cast<const void*>(&k_conv_thin<TE, PB, Epi>))) \
			return false; \
		hipLaunchKernelGGL((k_conv_thin<TE, PB, Epi>), grid, dim3(256), lds_bytes, stream, static_cast<const TE*>(x), static_cast<const TE*>(w), g, epi)
		switch (pb)
		{
			case 16:
				AVHIP_THIN(16);
				return true;
			case 8:
				AVHIP_THIN(8);
				return true;
			case 4:
				AVHIP_THIN(4);
				return true;
			case 2:
				if constexpr (sizeof(TE) <= 2)
				{
					AVHIP_THIN(2);
					return true;
				}
				return false;
			case 1:
				if constexpr (sizeof(TE) == 1)
				{
					AVHIP_THIN(1);
					return true;
				}
				return false;
			default:
				return false;
		}
#undef AVHIP_THIN
	}

#define AVHIP_INSTANTIATE(TE, EPI) template bool conv_thin_launch<TE, EPI>(hipStream_t, const avhipConvShape&, const void*, const void*, const EPI&);
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
