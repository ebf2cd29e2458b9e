/*
 * conv_winograd_fused.hip -- y = act(alpha1 * conv(x, w) + bias + alpha2 * z) + beta * y by Winograd F(2x2, 3x3) in ONE kernel.
 *
 * Replaces cuda_winogradFusedForward / kernel_winograd_fused (src/winograd_fused.cu:789,590 of the reference; header entry
 * cudaConvolutionWinogradFusedForward, include/Avocado/cuda_backend.h:840), a prototype that keeps an 8x8-pixel tile and
 * its transformed values in shared memory and multiplies on the scalar units.  Here the sixteen element-wise products of
 * the Winograd domain are sixteen small GEMMs on the matrix cores and nothing of the Winograd domain touches HBM:
 *
 *   workgroup  = 8 x 8 Winograd tiles (16 x 16 output pixels) of one image  x  128 filters, 4 wavefronts as 2 (tile rows) x 2
 *                (filters); a wavefront owns 32 tiles x 64 filters;
 *   input      : per block of 256 bytes of channels (128 fp16 / 64 fp32) the 18 x 18 pixel halo goes to LDS once (bf16 is
 *                converted to fp16 on the way: V must carry 11 mantissa bits to meet the 16-bit parity bar);
 *   for each of the 16 positions e = (ei, ej) of the transformed tile:
 *       A operand  V_e = (B^T d B)[ei][ej] is formed in registers from the FOUR halo pixels that B^T's two non-zeros per
 *                  row select (packed fp16 / fp32 adds), straight in the MFMA operand layout;
 *       B operand  U_e[k][c] comes from the pre-transformed weights [16, K, C] in global memory (L2 resident), fetched one
 *                  half-position ahead into registers, no LDS;
 *       M_e += V_e * U_e^T over the channel block on the matrix cores, then Y[a][b] += A^T[a][ei] * A^T[b][ej] * M_e
 *       (the output transform, linear, so it is applied per channel block);
 *   epilogue   : the four Y[a][b] accumulators leave through LDS as rows of 128 filters per output pixel, with the shared
 *                bias / residual / activation epilogue.
 *
 * The halo is stored as four parity planes (row parity, column parity): the tiles of a wavefront read, for a fixed patch
 * position, pixels two apart, which would alias LDS banks in a plain layout; inside a parity plane they are neighbours.
 * Entry pitch 272 bytes and row stride 9 * 272 - 16 make a 16-lane group (8 tile columns x 2 tile rows) hit all 64 banks.
 *
 * Tables (src/winograd_nonfused.cu:534-575): B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 -1 0 1], A^T = [1 .5 .5 0; 0 .5 -.5 1],
 * G unscaled (the weight transform kernel of winograd_transforms.hip produces U).
 * Limits: 3x3, stride 1, dilation 1, zero padding value, C a multiple of 8 (16-bit) or 4 (fp32), x and U below 2 GiB,
 * 16-bit inputs within the fp16 range.
 */
#include <utility>

#include "conv_epilogue.hpp"
#include "mfma_core.hpp"

namespace
{
	using namespace avhip;

	constexpr int TILE_BLOCK = 8; /* tiles per workgroup edge */
	constexpr int HALO = 2 * TILE_BLOCK + 2; /* 18 pixels */
	constexpr int PLANE_W = HALO / 2; /* entries per parity-plane row */
	constexpr int CHANNEL_BYTES = 256; /* bytes of channels per pixel and channel block */
	constexpr int PITCH = CHANNEL_BYTES + 16;
	constexpr int ROW_STRIDE = PLANE_W * PITCH - 16;
	constexpr int PLANE = (PLANE_W - 1) * ROW_STRIDE + PLANE_W * PITCH;
	constexpr int HALO_BYTES = 4 * PLANE;
	constexpr int HALO_ITEMS = HALO * HALO * (CHANNEL_BYTES / 16);
	constexpr int FUSED_BLOCK_N = 128;
	constexpr int PHASES = 32; /* 16 positions x 2 halves of the channel block */

	/* B^T row r = S0[r] * d[I0[r]] + S1[r] * d[I1[r]] */
	__host__ __device__ constexpr int bt_i0(int r) { return r == 0 ? 0 : 1; }
	__host__ __device__ constexpr int bt_i1(int r) { return r == 3 ? 3 : 2; }
	__host__ __device__ constexpr int bt_s0(int r) { return (r == 0 || r == 1) ? 1 : -1; }
	__host__ __device__ constexpr int bt_s1(int r) { return r == 0 ? -1 : 1; }
	/* A^T[a][i] */
	__host__ __device__ constexpr float at(int a, int i)
	{
		return a == 0 ? (i == 0 ? 1.0f : i == 3 ? 0.0f : 0.5f) : (i == 0 ? 0.0f : i == 1 ? 0.5f : i == 2 ? -0.5f : 1.0f);
	}

	typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
	template<typename TL> struct Lanes;
	template<> struct Lanes<f16_t>
	{
		typedef f16x8_t type;
	};
	template<> struct Lanes<float>
	{
		typedef f32x4_t type;
	};
	template<typename TX> struct Staged /* element type of the halo in LDS and of U */
	{
		typedef TX type;
	};
	template<> struct Staged<bf16_t>
	{
		typedef f16_t type;
	};

	struct FusedGeom
	{
		int H, W, C, K, Ho, Wo, pad_h, pad_w;
		int blocks_w, blocks_per_image; /* tile blocks across and per image */
		int images;
	};

	__device__ inline uint4 to_staged(uint4 v, bf16_t)
	{
		union
		{
			uint4 u;
			unsigned short s[8];
		} in;
		union
		{
			uint4 u;
			f16_t h[8];
		} out;
		in.u = v;
#pragma unroll
		for (int i = 0; i < 8; i++)
			out.h[i] = static_cast<f16_t>(__uint_as_float(static_cast<unsigned int>(in.s[i]) << 16));
		return out.u;
	}
	__device__ inline uint4 to_staged(uint4 v, f16_t)
	{
		return v;
	}
	__device__ inline uint4 to_staged(uint4 v, float)
	{
		return v;
	}

	template<typename TL, int S>
	__device__ __forceinline__ typename Lanes<TL>::type signed_of(const uint4 &raw)
	{
		union
		{
			uint4 u;
			typename Lanes<TL>::type v;
		} t;
		t.u = raw;
		return S > 0 ? t.v : -t.v;
	}

	template<typename TX, int ACT>
	struct FusedKernel
	{
		typedef typename Staged<TX>::type TL;
		typedef typename Mma<TL>::acc_t acc_t;

		const char *lds;
		__amdgpu_buffer_rsrc_t u_rsrc;
		int a_base; /* this lane's LDS byte offset of (its tile, patch (0,0), its half of a slab) */
		unsigned int u_lane[2]; /* byte offset of this lane's U rows (two filter tiles), OUT_OF_RANGE when the filter does not exist */
		unsigned int u_half; /* 0 or 16: which half of a 32-byte slab this lane supplies */
		unsigned int u_position_bytes; /* K * C * sizeof(TL) */
		unsigned int c_bytes; /* C * sizeof(TL) */
		acc_t Y[2][2][2], M[2];
		uint4 a_raw[2][4]; /* two slabs in flight x the four pixels of a position */
		uint4 b_raw[2][4][2]; /* two phases in flight x 4 slabs x 2 filter tiles */

		/* LDS offset of halo pixel (i, j) of a tile relative to the tile's own (0, 0) pixel */
		__device__ static constexpr int patch_offset(int i, int j)
		{
			return ((i & 1) * 2 + (j & 1)) * PLANE + (i >> 1) * ROW_STRIDE + (j >> 1) * PITCH;
		}
		template<int P>
		__device__ __forceinline__ void fetch_b(int channel_block)
		{
			constexpr int E = (P % PHASES) / 2, HALF = P % 2;
			const unsigned int base = E * u_position_bytes + channel_block * CHANNEL_BYTES + HALF * 128 + u_half;
#pragma unroll
			for (int s = 0; s < 4; s++)
			{
				const bool in_c = channel_block * CHANNEL_BYTES + HALF * 128 + s * 32 + u_half < c_bytes;
#pragma unroll
				for (int tn = 0; tn < 2; tn++)
					b_raw[P % 2][s][tn] = buffer_fetch(u_rsrc, (in_c && u_lane[tn] != OUT_OF_RANGE) ? u_lane[tn] + base + s * 32 : OUT_OF_RANGE);
			}
		}
		template<int P, int SLAB>
		__device__ __forceinline__ void read_a()
		{
			constexpr int E = P / 2, HALF = P % 2, EI = E / 4, EJ = E % 4;
			constexpr int byte = HALF * 128 + SLAB * 32;
			const char *p = lds + a_base + byte;
			a_raw[SLAB % 2][0] = *reinterpret_cast<const uint4*>(p + patch_offset(bt_i0(EI), bt_i0(EJ)));
			a_raw[SLAB % 2][1] = *reinterpret_cast<const uint4*>(p + patch_offset(bt_i0(EI), bt_i1(EJ)));
			a_raw[SLAB % 2][2] = *reinterpret_cast<const uint4*>(p + patch_offset(bt_i1(EI), bt_i0(EJ)));
			a_raw[SLAB % 2][3] = *reinterpret_cast<const uint4*>(p + patch_offset(bt_i1(EI), bt_i1(EJ)));
		}
		template<int P, int SLAB>
		__device__ __forceinline__ void multiply()
		{
			constexpr int E = P / 2, EI = E / 4, EJ = E % 4;
			typedef typename Lanes<TL>::type V;
			union
			{
				V v;
				Chunk c;
			} a;
			const V r0 = signed_of<TL, bt_s0(EJ)>(a_raw[SLAB % 2][0]) + signed_of<TL, bt_s1(EJ)>(a_raw[SLAB % 2][1]);
			const V r1 = signed_of<TL, bt_s0(EJ)>(a_raw[SLAB % 2][2]) + signed_of<TL, bt_s1(EJ)>(a_raw[SLAB % 2][3]);
			a.v = (bt_s0(EI) > 0 ? r0 : -r0) + (bt_s1(EI) > 0 ? r1 : -r1);
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
			{
				Chunk b;
				b.u = b_raw[P % 2][SLAB][tn];
				Mma<TL>::run(a.c, b, M[tn]);
			}
		}
		template<int E>
		__device__ __forceinline__ void fold()
		{
			constexpr int EI = E / 4, EJ = E % 4;
#pragma unroll
			for (int a = 0; a < 2; a++)
#pragma unroll
				for (int b = 0; b < 2; b++)
				{
					const float coefficient = at(a, EI) * at(b, EJ);
					if (coefficient != 0.0f)
					{
#pragma unroll
						for (int tn = 0; tn < 2; tn++)
#pragma unroll
							for (int v = 0; v < 16; v++)
								Y[a][b][tn][v] += coefficient * M[tn][v];
					}
				}
#pragma unroll
			for (int tn = 0; tn < 2; tn++)
#pragma unroll
				for (int v = 0; v < 16; v++)
					M[tn][v] = 0;
		}
		/* one half of one position: U for the next phase is requested first, LDS reads run one slab ahead of the MFMAs */
		template<int P>
		__device__ __forceinline__ void phase(int channel_block)
		{
			if (P + 1 < PHASES)
				fetch_b<P + 1>(channel_block);
			else
				fetch_b<PHASES>(channel_block + 1); /* wraps to phase 0 of the next channel block (zeros past the last) */
			if (P == 0)
				read_a<P, 0>();
			read_a<P, 1>();
			multiply<P, 0>();
			read_a<P, 2>();
			multiply<P, 1>();
			read_a<P, 3>();
			multiply<P, 2>();
			if (P + 1 < PHASES)
				read_a<(P + 1) % PHASES, 0>();
			multiply<P, 3>();
			if (P % 2 == 1)
				fold<P / 2>();
			/* the 32 phases are one basic block: without a fence the scheduler hoists the loads of many phases and spills */
			__builtin_amdgcn_sched_barrier(0);
		}
		template<int ... Ps>
		__device__ __forceinline__ void all_phases(int channel_block, std::integer_sequence<int, Ps...>)
		{
			(phase<Ps>(channel_block), ...);
		}
	};

	template<typename TX, int ACT>
	__global__ __launch_bounds__(256, 1) void k_winograd_fused(const TX *__restrict__ x, const void *__restrict__ U, FusedGeom g, FloatEpilogue<TX> epi)
	{
		typedef FusedKernel<TX, ACT> Kernel;
		typedef typename Kernel::TL TL;
		__shared__ __attribute__((aligned(16))) char lds[HALO_BYTES];
		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wm = wave >> 1, wn = wave & 1;

		/* which 8 x 8 tile block of which image, which 128 filters */
		const int image = blockIdx.x / g.blocks_per_image;
		const int in_image = blockIdx.x - image * g.blocks_per_image;
		const int block_h = in_image / g.blocks_w, block_w = in_image - block_h * g.blocks_w;
		const int k0 = blockIdx.y * FUSED_BLOCK_N;
		const int k = k0 + drain_column<2>();
		typename FloatEpilogue<TX>::Columns columns;
		epi.load_columns(k, columns);
		epi.pin();

		Kernel kn;
		kn.lds = lds;
		kn.c_bytes = g.C * sizeof(TL);
		kn.u_position_bytes = static_cast<unsigned int>(g.K) * kn.c_bytes;
		kn.u_rsrc = make_buffer(U, 16u * kn.u_position_bytes);
		kn.u_half = (lane >> 5) * 16;
		const int r = lane & 31;
		kn.a_base = (4 * wm + (r >> 3)) * ROW_STRIDE + (r & 7) * PITCH + (lane >> 5) * 16;
#pragma unroll
		for (int tn = 0; tn < 2; tn++)
		{
			const int row = k0 + wn * 64 + tn * 32 + r;
			kn.u_lane[tn] = row < g.K ? static_cast<unsigned int>(row) * kn.c_bytes : OUT_OF_RANGE;
		}
#pragma unroll
		for (int a = 0; a < 2; a++)
#pragma unroll
			for (int b = 0; b < 2; b++)
#pragma unroll
				for (int tn = 0; tn < 2; tn++)
#pragma unroll
					for (int v = 0; v < 16; v++)
						kn.Y[a][b][tn][v] = 0;
#pragma unroll
		for (int tn = 0; tn < 2; tn++)
#pragma unroll
			for (int v = 0; v < 16; v++)
				kn.M[tn][v] = 0;

		const __amdgpu_buffer_rsrc_t x_rsrc = make_buffer(x, static_cast<unsigned int>(static_cast<int64_t>(g.images) * g.H * g.W * g.C * sizeof(TX)));
		const int ih0 = 2 * TILE_BLOCK * block_h + g.pad_h, iw0 = 2 * TILE_BLOCK * block_w + g.pad_w;
		const int channel_blocks = (g.C * static_cast<int>(sizeof(TL)) + CHANNEL_BYTES - 1) / CHANNEL_BYTES;

		kn.template fetch_b<0>(0);
		for (int cb = 0; cb < channel_blocks; cb++)
		{
			__syncthreads(); /* the previous block's halo has been read by everyone */
			constexpr int ROUNDS = (HALO_ITEMS + 255) / 256;
			constexpr int BATCH = 7;
			static_assert(ROUNDS % BATCH == 0, "halo rounds are issued in equal batches");
#pragma unroll
			for (int batch = 0; batch < ROUNDS / BATCH; batch++)
			{
				uint4 v[BATCH];
#pragma unroll
				for (int i = 0; i < BATCH; i++)
				{
					const int item = (batch * BATCH + i) * 256 + tid;
					const int pixel = item >> 4, chunk = item & 15;
					const int hy = pixel / HALO, hx = pixel - hy * HALO;
					const int ih = ih0 + hy, iw = iw0 + hx;
					const int c_byte = cb * CHANNEL_BYTES + chunk * 16;
					const bool exists = item < HALO_ITEMS && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W && c_byte < static_cast<int>(kn.c_bytes);
					const unsigned int off = static_cast<unsigned int>((image * g.H + ih) * g.W + iw) * kn.c_bytes + c_byte;
					v[i] = buffer_fetch(x_rsrc, exists ? off : OUT_OF_RANGE);
				}
#pragma unroll
				for (int i = 0; i < BATCH; i++)
				{
					const int item = (batch * BATCH + i) * 256 + tid;
					const int pixel = item >> 4, chunk = item & 15;
					const int hy = pixel / HALO, hx = pixel - hy * HALO;
					if (item < HALO_ITEMS)
						*reinterpret_cast<uint4*>(lds + ((hy & 1) * 2 + (hx & 1)) * PLANE + (hy >> 1) * ROW_STRIDE + (hx >> 1) * PITCH + chunk * 16) = to_staged(v[i], TX());
				}
			}
			__syncthreads();
			kn.all_phases(cb, std::make_integer_sequence<int, PHASES>());
		}

		/* four output pixels per tile: each (a, b) plane of accumulators leaves like one GEMM tile of 64 rows x 128 columns */
		const int64_t image_pixels = static_cast<int64_t>(image) * g.Ho * g.Wo;
		auto leave = [&](auto row_of_four, auto column_of_four) __attribute__((always_inline))
		{
			constexpr int a = decltype(row_of_four)::value, b = decltype(column_of_four)::value;
			typename Kernel::acc_t plane[1][2] = { { kn.Y[a][b][0], kn.Y[a][b][1] } };
			auto row_out = [&](int row, const float (&v)[4], int) __attribute__((always_inline))
			{
				const int th = TILE_BLOCK * block_h + (row >> 3), tw = TILE_BLOCK * block_w + (row & 7);
				const int oh = 2 * th + a, ow = 2 * tw + b;
				if (oh < g.Ho && ow < g.Wo && k < g.K)
					epi.template store<ACT>(image_pixels + static_cast<int64_t>(oh) * g.Wo + ow, k, v, columns);
			};
			/* the long epilogue of ACT_ANY once per plane, in a loop over its rows; unrolled per row, the four planes were no
			 * longer unrolled themselves and the accumulators went to scratch memory */
			if constexpr (ACT == ACT_ANY)
				drain_tile_rolled<TL, 1, 2>(lds, plane, row_out);
			else
				drain_tile<TL, 1, 2>(lds, plane, row_out);
		};
		typedef std::integral_constant<int, 0> zero_t;
		typedef std::integral_constant<int, 1> one_t;
		leave(zero_t(), zero_t());
		leave(zero_t(), one_t());
		leave(one_t(), zero_t());
		leave(one_t(), one_t());
	}

	template<typename TX>
	int launch(hipStream_t st, const avhipConvShape &s, const void *x, const void *U, const void *bias, const void *z, void *y, double alpha1, double alpha2,
			double beta, int activation)
	{
		typedef typename Staged<TX>::type TL;
		const int chunk = 16 / static_cast<int>(sizeof(TX));
		if (s.C % chunk != 0 || !aligned_to(x, 16) || !aligned_to(U, 16))
			return AVHIP_NOT_SUPPORTED;
		const int64_t x_bytes = static_cast<int64_t>(s.N) * s.H * s.W * s.C * sizeof(TX);
		const int64_t u_bytes = static_cast<int64_t>(16) * s.K * s.C * sizeof(TL);
		if (x_bytes >= (1ll << 31) || u_bytes >= (1ll << 31))
			return AVHIP_NOT_SUPPORTED;
		FusedGeom g;
		g.H = s.H;
		g.W = s.W;
		g.C = s.C;
		g.K = s.K;
		g.Ho = s.Ho;
		g.Wo = s.Wo;
		g.pad_h = s.pad_h;
		g.pad_w = s.pad_w;
		g.images = s.N;
		const int tiles_h = (s.Ho + 1) / 2, tiles_w = (s.Wo + 1) / 2;
		g.blocks_w = (tiles_w + TILE_BLOCK - 1) / TILE_BLOCK;
		g.blocks_per_image = g.blocks_w * ((tiles_h + TILE_BLOCK - 1) / TILE_BLOCK);
		const int64_t blocks = static_cast<int64_t>(s.N) * g.blocks_per_image;
		const int64_t filter_blocks = (s.K + FUSED_BLOCK_N - 1) / FUSED_BLOCK_N;
		if (blocks >= (1ll << 31) || filter_blocks > 65535)
			return AVHIP_NOT_SUPPORTED;
		const bool vec = s.K % 4 == 0 && aligned_to(y, 4 * sizeof(TX)) && (z == nullptr || aligned_to(z, 4 * sizeof(TX)));
		const FloatEpilogue<TX> epi { static_cast<const float*>(bias), static_cast<const TX*>(z), static_cast<TX*>(y), static_cast<float>(alpha1),
				static_cast<float>(alpha2), static_cast<float>(beta), activation, s.K, vec };
		const dim3 grid(static_cast<unsigned int>(blocks), static_cast<unsigned int>(filter_blocks));
		if (is_simple_activation(activation))
			hipLaunchKernelGGL((k_winograd_fused<TX, ACT_SIMPLE>), grid, dim3(256), 0, st, static_cast<const TX*>(x), U, g, epi);
		else
			hipLaunchKernelGGL((k_winograd_fused<TX, ACT_ANY>), grid, dim3(256), 0, st, static_cast<const TX*>(x), U, g, epi);
		return 0;
	}
}

extern "C" int avhip_conv2d_winograd_fused(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias,
		const void *z, void *y, double alpha1, double alpha2, double beta, int activation)
{
	if (shape == nullptr || x == nullptr || U == nullptr || y == nullptr)
		return AVHIP_BAD_PARAM;
	const avhipConvShape &s = *shape;
	if (s.N <= 0 || s.H <= 0 || s.W <= 0 || s.C <= 0 || s.K <= 0 || s.Ho <= 0 || s.Wo <= 0)
		return AVHIP_BAD_PARAM;
	if (s.R != 3 || s.S != 3 || s.stride_h != 1 || s.stride_w != 1 || s.dil_h != 1 || s.dil_w != 1)
		return AVHIP_NOT_SUPPORTED;
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (dtype)
	{
		case DT_FLOAT32:
			return launch<float>(st, s, x, U, bias, z, y, alpha1, alpha2, beta, activation);
		case DT_FLOAT16:
			return launch<f16_t>(st, s, x, U, bias, z, y, alpha1, alpha2, beta, activation);
		case DT_BFLOAT16:
			return launch<bf16_t>(st, s, x, U, bias, z, y, alpha1, alpha2, beta, activation);
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}
