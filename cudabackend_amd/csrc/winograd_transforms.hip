/*
 * winograd_transforms.hip -- the non-fused Winograd transforms for F(2x2,3x3), F(4x4,3x3) and F(2x2,5x5): weight, input and
 * output for the forward pass, gradient and update for the weight gradient.
 *
 * Replaces kernel_winograd_{weight,input,output,gradient,update}_transform and their launchers of the reference
 * (src/winograd_nonfused.cu:257-519, 609-877).  The mathematics is the same sandwich product M * tile * M^T with the
 * same coefficient tables (src/winograd_nonfused.cu:534-575); the mapping to the machine is not:
 *
 *  - these kernels are HBM-bound, so one work-item owns one tile x one 16-byte (or 8-byte) vector of channels, issues
 *    all t*t vector loads up front, transforms in registers and writes t*t vectors.  A 64-wide wavefront therefore reads
 *    and writes whole 512- or 1024-byte channel rows, and consecutive wavefronts walk consecutive tiles of one matrix plane;
 *  - the coefficient tables are compile-time constants: zero terms disappear and +-1 terms become adds when the loops are
 *    unrolled, so there is no table upload, no LDS and no data-dependent branch;
 *  - overlapping tile halos are served by L2 / Infinity Cache, not staged through LDS;
 *  - the matrix dtype is independent of the tensor dtype (fp16 or fp32 matrices for 16-bit tensors keep F(4x4,3x3) usable);
 *  - 16-bit values are computed in fp32 and rounded to nearest even on store.
 */
#include <type_traits>

#include "conv_epilogue.hpp"
#include "mfma_core.hpp"

namespace
{
	using namespace avhip;

	/* Coefficient tables (row-major).  which: 0 = G [t x r], 1 = B^T [t x t], 2 = A^T [m x t], 3 = gradient [t x m],
	 * 4 = update [r x t]. */
	template<int M, int R> struct Tab;
	template<> struct Tab<2, 3>
	{
		__host__ __device__ static constexpr double get(int which, int i, int j)
		{
			constexpr double G[4 * 3] = { 1, 0, 0, 1, 1, 1, 1, -1, 1, 0, 0, 1 };
			constexpr double BT[4 * 4] = { 1, 0, -1, 0, 0, 1, 1, 0, 0, -1, 1, 0, 0, -1, 0, 1 };
			constexpr double AT[2 * 4] = { 1, 0.5, 0.5, 0, 0, 0.5, -0.5, 1 };
			constexpr double GR[4 * 2] = { 1, 0, 1, 1, 1, -1, 0, 1 };
			constexpr double UP[3 * 4] = { 1, 0.5, 0.5, 0, 0, 0.5, -0.5, 0, 0, 0.5, 0.5, 1 };
			return which == 0 ? G[i * 3 + j] : which == 1 ? BT[i * 4 + j] : which == 2 ? AT[i * 4 + j] : which == 3 ? GR[i * 2 + j] : UP[i * 4 + j];
		}
	};
	template<> struct Tab<4, 3>
	{
		__host__ __device__ static constexpr double get(int which, int i, int j)
		{
			constexpr double a = 1.0 / 3.0;
			constexpr double G[6 * 3] = { 1, 0, 0, 2 * a, 2 * a, 2 * a, 2 * a, -2 * a, 2 * a, a, 2 * a, 4 * a, a, -2 * a, 4 * a, 0, 0, 2 };
			constexpr double BT[6 * 6] = { 1, 0, -1.25, 0, 0.25, 0, 0, 1, 1, -0.25, -0.25, 0, 0, -1, 1, 0.25, -0.25, 0, 0, -1, -0.5, 1, 0.5, 0, 0, 1, -0.5,
					-1, 0.5, 0, 0, 1, 0, -1.25, 0, 0.25 };
			constexpr double AT[4 * 6] = { 1, 1, 1, 0.25, 0.25, 0, 0, 1, -1, 0.5, -0.5, 0, 0, 1, 1, 1, 1, 0, 0, 1, -1, 2, -2, 2 };
			constexpr double GR[6 * 4] = { 1, 0, 0, 0, 2 * a, 2 * a, 2 * a, 2 * a, 2 * a, -2 * a, 2 * a, -2 * a, a, 2 * a, 4 * a, 8 * a, a, -2 * a, 4 * a, -8 * a, 0,
					0, 0, 2 };
			constexpr double UP[3 * 6] = { 1, 1, 1, 0.25, 0.25, 0, 0, 1, -1, 0.5, -0.5, 0, 0, 1, 1, 1, 1, 2 };
			return which == 0 ? G[i * 3 + j] : which == 1 ? BT[i * 6 + j] : which == 2 ? AT[i * 6 + j] : which == 3 ? GR[i * 4 + j] : UP[i * 6 + j];
		}
	};
	template<> struct Tab<2, 5>
	{
		__host__ __device__ static constexpr double get(int which, int i, int j)
		{
			constexpr double a = 1.0 / 3.0;
			constexpr double G[6 * 5] = { 1, 0, 0, 0, 0, 2 * a, 2 * a, 2 * a, 2 * a, 2 * a, 2 * a, -2 * a, 2 * a, -2 * a, 2 * a, a / 2, a, 2 * a, 4 * a, 8 * a,
					a / 2, -a, 2 * a, -4 * a, 8 * a, 0, 0, 0, 0, 2 };
			constexpr double BT[6 * 6] = { 1, 0, -1.25, 0, 0.25, 0, 0, 1, 1, -0.25, -0.25, 0, 0, -1, 1, 0.25, -0.25, 0, 0, -1, -0.5, 1, 0.5, 0, 0, 1, -0.5,
					-1, 0.5, 0, 0, 1, 0, -1.25, 0, 0.25 };
			constexpr double AT[2 * 6] = { 1, 1, 1, 0.5, 0.5, 0, 0, 1, -1, 1, -1, 2 };
			constexpr double GR[6 * 2] = { 1, 0, 2 * a, 2 * a, 2 * a, -2 * a, a, 2 * a, a, -2 * a, 0, 1 };
			constexpr double UP[5 * 6] = { 1, 1, 1, 0.25, 0.25, 0, 0, 1, -1, 0.5, -0.5, 0, 0, 1, 1, 1, 1, 0, 0, 1, -1, 2, -2, 0, 0, 1, 1, 4, 4, 4 };
			return which == 0 ? G[i * 5 + j] : which == 1 ? BT[i * 6 + j] : which == 2 ? AT[i * 6 + j] : which == 3 ? GR[i * 2 + j] : UP[i * 6 + j];
		}
	};

	/* acc (+)= c * d with the coefficient known at compile time once the caller's loops are unrolled. */
	template<typename CT, int V>
	__device__ inline void axpy(bool &have, CT (&acc)[V], double c, const CT (&d)[V])
	{
		if (c == 0.0)
			return;
#pragma unroll
		for (int v = 0; v < V; v++)
		{
			const CT term = (c == 1.0) ? d[v] : (c == -1.0) ? -d[v] : static_cast<CT>(c) * d[v];
			acc[v] = have ? acc[v] + term : term;
		}
		have = true;
	}

	/* out[ROWS x ROWS] = Mx[ROWS x COLS] * d[COLS x COLS] * Mx^T, Mx = table `WHICH` of Tab<M, R>. */
	template<int M, int R, int WHICH, int ROWS, int COLS, typename CT, int V>
	__device__ inline void sandwich(const CT (&d)[COLS * COLS][V], CT (&out)[ROWS * ROWS][V])
	{
		CT tmp[ROWS * COLS][V];
#pragma unroll
		for (int i = 0; i < ROWS; i++)
#pragma unroll
			for (int j = 0; j < COLS; j++)
			{
				bool have = false;
#pragma unroll
				for (int k = 0; k < COLS; k++)
					axpy<CT, V>(have, tmp[i * COLS + j], Tab<M, R>::get(WHICH, i, k), d[k * COLS + j]);
				if (!have)
				{
#pragma unroll
					for (int v = 0; v < V; v++)
						tmp[i * COLS + j][v] = static_cast<CT>(0);
				}
			}
#pragma unroll
		for (int i = 0; i < ROWS; i++)
#pragma unroll
			for (int j = 0; j < ROWS; j++)
			{
				bool have = false;
#pragma unroll
				for (int k = 0; k < COLS; k++)
					axpy<CT, V>(have, out[i * ROWS + j], Tab<M, R>::get(WHICH, j, k), tmp[i * COLS + k]);
				if (!have)
				{
#pragma unroll
					for (int v = 0; v < V; v++)
						out[i * ROWS + j][v] = static_cast<CT>(0);
				}
			}
	}

	template<int M, int R, typename T, typename TM, int V>
	__global__ __launch_bounds__(256) void k_weight_transform(const T *__restrict__ w, TM *__restrict__ U, int K, int C, int invert)
	{
		typedef typename Traits<T>::compute CT;
		constexpr int t = M + R - 1;
		const int CV = (C + V - 1) / V;
		const size_t gid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
		const int cv = static_cast<int>(gid % CV);
		const size_t k = gid / CV;
		if (k >= static_cast<size_t>(K))
			return;
		const int c = cv * V;
		const int valid = C - c;

		CT g[R * R][V];
#pragma unroll
		for (int i = 0; i < R; i++)
#pragma unroll
			for (int j = 0; j < R; j++)
			{
				const int si = invert ? (R - 1 - i) : i;
				const int sj = invert ? (R - 1 - j) : j;
				load_vec<T, V, CT>(w + ((k * R + si) * R + sj) * C + c, valid, g[i * R + j]);
			}
		CT out[t * t][V];
		sandwich<M, R, 0, t, R, CT, V>(g, out);
#pragma unroll
		for (int i = 0; i < t * t; i++)
		{
			typename Traits<TM>::compute o[V];
#pragma unroll
			for (int v = 0; v < V; v++)
				o[v] = static_cast<typename Traits<TM>::compute>(out[i][v]);
			store_vec<TM, V>(U + (static_cast<size_t>(i) * K + k) * C + c, valid, o);
		}
	}

	/* IDX is the integer type of the work-item and tile indices: 32 bits whenever the problem allows it (64-bit divisions
	 * cost more than the transform itself).  V > 1 instances are launched only when every vector is complete and aligned:
	 * they have no tail handling, and outside the image they load from a clamped address and select the padding value, so
	 * the whole work-item is branch-free and all its loads are in flight together. */
	/* BUF instances (complete vectors of 4, 8 or 16 bytes, zero padding value, x below 2 GiB) fetch through a buffer descriptor: a pixel outside the image is
	 * asked for at an out-of-range offset and comes back as zeros, so every load of the work-item is unconditional.  With ordinary
	 * loads the compiler turns "load at a clamped address, then select the padding value" back into a branch around each load,
	 * and where the element conversion is an instruction of its own (fp16) it ends up behind the branch with a wait in front of it: the
	 * sixteen loads of a tile then run one after the other (the fp16 instance was 13 % slower than the bf16 one on the same bytes). */
	template<int M, int R, typename T, typename TM, int V, typename IDX, bool BUF = false>
	__global__ __launch_bounds__(256) void k_input_transform(const T *__restrict__ x, TM *__restrict__ Vm, int N, int H, int W, int C, int Th, int Tw,
			int pad_h, int pad_w, typename Traits<T>::compute padv)
	{
		typedef typename Traits<T>::compute CT;
		constexpr int t = M + R - 1;
		constexpr bool FULL = V > 1;
		static_assert(!BUF || (FULL && (sizeof(T) * V == 4 || sizeof(T) * V == 8 || sizeof(T) * V == 16) && sizeof(IDX) == 4), "whole 4-, 8- or 16-byte vectors, 32-bit offsets");
		const IDX CV = static_cast<IDX>((C + V - 1) / V);
		const IDX tiles = static_cast<IDX>(N) * Th * Tw;
		/* neighbouring tiles share input pixels: consecutive runs of tiles go to one XCD, whose L2 then serves the overlap */
		const IDX gid = static_cast<IDX>(xcd_block(blockIdx.x, gridDim.x)) * 256 + threadIdx.x;
		const IDX tile = gid / CV;
		const int cv = static_cast<int>(gid - tile * CV);
		if (tile >= tiles)
			return;
		const IDX row = tile / static_cast<IDX>(Tw);
		const int tw = static_cast<int>(tile - row * Tw);
		const IDX n = row / static_cast<IDX>(Th);
		const int th = static_cast<int>(row - n * Th);
		const int c = cv * V;
		const int valid = FULL ? V : C - c;
		const int ih0 = pad_h + th * M, iw0 = pad_w + tw * M;
		const T *image = x + static_cast<size_t>(n) * H * W * C + c;
		typedef typename std::conditional<sizeof(IDX) == 4, int, int64_t>::type OFF; /* offsets inside one image */

		CT d[t * t][V];
		if constexpr (BUF)
		{
			const __amdgpu_buffer_rsrc_t rx = make_buffer(x, static_cast<unsigned int>(N) * H * W * C * static_cast<unsigned int>(sizeof(T)));
			const unsigned int base = (static_cast<unsigned int>(n) * H * W * C + c) * static_cast<unsigned int>(sizeof(T));
			Pack<T, V> raw[t * t];
#pragma unroll
			for (int a = 0; a < t; a++)
#pragma unroll
				for (int b = 0; b < t; b++)
				{
					const int ih = ih0 + a, iw = iw0 + b;
					const bool inside = (static_cast<unsigned int>(ih) < static_cast<unsigned int>(H)) & (static_cast<unsigned int>(iw) < static_cast<unsigned int>(W));
					const unsigned int offset = inside ? base + static_cast<unsigned int>((ih * W + iw) * C) * static_cast<unsigned int>(sizeof(T)) : OUT_OF_RANGE;
					if constexpr (sizeof(T) * V == 16)
						raw[a * t + b] = __builtin_bit_cast(Pack<T, V>, __builtin_amdgcn_raw_buffer_load_b128(rx, static_cast<int>(offset), 0, 0));
					else if constexpr (sizeof(T) * V == 8)
						raw[a * t + b] = __builtin_bit_cast(Pack<T, V>, __builtin_amdgcn_raw_buffer_load_b64(rx, static_cast<int>(offset), 0, 0));
					else
						raw[a * t + b] = __builtin_bit_cast(Pack<T, V>, __builtin_amdgcn_raw_buffer_load_b32(rx, static_cast<int>(offset), 0, 0));
				}
#pragma unroll
			for (int i = 0; i < t * t; i++)
#pragma unroll
				for (int v = 0; v < V; v++)
					d[i][v] = Traits<T>::load(raw[i].v[v]);
		}
		else
#pragma unroll
		for (int a = 0; a < t; a++)
#pragma unroll
			for (int b = 0; b < t; b++)
			{
				const int ih = ih0 + a;
				const int iw = iw0 + b;
				const bool inside = ih >= 0 && ih < H && iw >= 0 && iw < W;
				if (FULL)
				{
					load_vec<T, V, CT>(image + (inside ? (static_cast<OFF>(ih) * W + iw) * C : 0), V, d[a * t + b]);
#pragma unroll
					for (int v = 0; v < V; v++)
						d[a * t + b][v] = inside ? d[a * t + b][v] : padv;
				}
				else if (inside)
					load_vec<T, V, CT>(image + (static_cast<size_t>(ih) * W + iw) * C, valid, d[a * t + b]);
				else
				{
#pragma unroll
					for (int v = 0; v < V; v++)
						d[a * t + b][v] = padv;
				}
			}
		CT out[t * t][V];
		sandwich<M, R, 1, t, t, CT, V>(d, out);
#pragma unroll
		for (int i = 0; i < t * t; i++)
		{
			typename Traits<TM>::compute o[V];
#pragma unroll
			for (int v = 0; v < V; v++)
				o[v] = static_cast<typename Traits<TM>::compute>(out[i][v]);
			store_vec<TM, V, typename Traits<TM>::compute, FULL>(Vm + (static_cast<size_t>(i) * tiles + tile) * C + c, valid, o);
		}
	}

	template<int M, int R, typename T, typename TM, int V, int ACT, typename IDX>
	__global__ __launch_bounds__(256) void k_output_transform(const TM *__restrict__ Mx, T *y, const typename Traits<T>::compute *__restrict__ bias,
			const T *z, int N, int H, int W, int K, int Th, int Tw, typename Traits<T>::compute alpha1, typename Traits<T>::compute alpha2,
			typename Traits<T>::compute beta, int activation)
	{
		typedef typename Traits<T>::compute CT;
		constexpr int t = M + R - 1;
		constexpr bool FULL = V > 1;
		const IDX KV = static_cast<IDX>((K + V - 1) / V);
		const IDX tiles = static_cast<IDX>(N) * Th * Tw;
		const IDX gid = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x;
		const IDX tile = gid / KV;
		const int kv = static_cast<int>(gid - tile * KV);
		if (tile >= tiles)
			return;
		const IDX row = tile / static_cast<IDX>(Tw);
		const int tw = static_cast<int>(tile - row * Tw);
		const IDX n = row / static_cast<IDX>(Th);
		const int th = static_cast<int>(row - n * Th);
		const int k = kv * V;
		const int valid = FULL ? V : K - k;

		CT d[t * t][V];
#pragma unroll
		for (int i = 0; i < t * t; i++)
		{
			typename Traits<TM>::compute tmp[V];
			load_vec<TM, V>(Mx + (static_cast<size_t>(i) * tiles + tile) * K + k, valid, tmp);
#pragma unroll
			for (int v = 0; v < V; v++)
				d[i][v] = static_cast<CT>(tmp[v]);
		}
		CT bv[V];
#pragma unroll
		for (int v = 0; v < V; v++)
			bv[v] = (bias != nullptr && v < valid) ? bias[k + v] : static_cast<CT>(0);
		CT out[M * M][V];
		sandwich<M, R, 2, M, t, CT, V>(d, out);

		const size_t image = static_cast<size_t>(n) * H * W;
#pragma unroll
		for (int a = 0; a < M; a++)
#pragma unroll
			for (int b = 0; b < M; b++)
			{
				const int oh = th * M + a;
				const int ow = tw * M + b;
				if (oh < H && ow < W)
				{
					const size_t idx = (image + static_cast<size_t>(oh * W + ow)) * K + k;
					CT r[V];
#pragma unroll
					for (int v = 0; v < V; v++)
						r[v] = alpha1 * out[a * M + b][v] + bv[v];
					if (z != nullptr)
					{
						CT zv[V];
						load_vec<T, V, CT>(z + idx, valid, zv);
#pragma unroll
						for (int v = 0; v < V; v++)
							r[v] += alpha2 * zv[v];
					}
#pragma unroll
					for (int v = 0; v < V; v++)
						r[v] = activate<ACT, CT>(activation, r[v]);
					if (beta != static_cast<CT>(0))
					{
						CT yv[V];
						load_vec<T, V, CT>(y + idx, valid, yv);
#pragma unroll
						for (int v = 0; v < V; v++)
							r[v] += beta * yv[v];
					}
					store_vec<T, V, CT, FULL>(y + idx, valid, r);
				}
			}
	}

	/* Weight-gradient side, first transform: one M x M tile of dy (tiles do not overlap, positions past the border are zero)
	 * becomes G' dy G'^T, a t x t tile of the matrices [t*t, tiles, K] (src/winograd_nonfused.cu:425-474). */
	template<int M, int R, typename T, typename TM, int V>
	__global__ __launch_bounds__(256) void k_gradient_transform(const T *__restrict__ dy, TM *__restrict__ Mx, int N, int H, int W, int K, int Th, int Tw)
	{
		typedef typename Traits<T>::compute CT;
		constexpr int t = M + R - 1;
		const size_t KV = static_cast<size_t>((K + V - 1) / V);
		const size_t tiles = static_cast<size_t>(N) * Th * Tw;
		const size_t gid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
		const size_t tile = gid / KV;
		if (tile >= tiles)
			return;
		const int k = static_cast<int>(gid - tile * KV) * V;
		const int valid = K - k;
		const size_t row = tile / Tw;
		const int tw = static_cast<int>(tile - row * Tw);
		const size_t n = row / Th;
		const int th = static_cast<int>(row - n * Th);

		CT d[M * M][V];
#pragma unroll
		for (int a = 0; a < M; a++)
#pragma unroll
			for (int b = 0; b < M; b++)
			{
				const int h = th * M + a, w = tw * M + b;
				if (h < H && w < W)
					load_vec<T, V, CT>(dy + ((n * H + h) * W + w) * K + k, valid, d[a * M + b]);
				else
				{
#pragma unroll
					for (int v = 0; v < V; v++)
						d[a * M + b][v] = static_cast<CT>(0);
				}
			}
		CT out[t * t][V];
		sandwich<M, R, 3, t, M, CT, V>(d, out);
#pragma unroll
		for (int i = 0; i < t * t; i++)
		{
			typename Traits<TM>::compute o[V];
#pragma unroll
			for (int v = 0; v < V; v++)
				o[v] = static_cast<typename Traits<TM>::compute>(out[i][v]);
			store_vec<TM, V>(Mx + (static_cast<size_t>(i) * tiles + tile) * K + k, valid, o);
		}
	}

	/* Weight-gradient side, last transform: dw[k, :, :, c] = alpha * U' m U'^T + beta * dw, m = the t x t tile of the matrices
	 * [t*t, K, C] at (k, c) (src/winograd_nonfused.cu:475-519). */
	template<int M, int R, typename T, typename TM, int V>
	__global__ __launch_bounds__(256) void k_update_transform(const TM *__restrict__ Mx, T *dw, int K, int C, typename Traits<T>::compute alpha,
			typename Traits<T>::compute beta)
	{
		typedef typename Traits<T>::compute CT;
		constexpr int t = M + R - 1;
		const int CV = (C + V - 1) / V;
		const size_t gid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
		const int c = static_cast<int>(gid % CV) * V;
		const size_t k = gid / CV;
		if (k >= static_cast<size_t>(K))
			return;
		const int valid = C - c;

		CT m[t * t][V];
#pragma unroll
		for (int i = 0; i < t * t; i++)
			load_vec<TM, V, CT>(Mx + (static_cast<size_t>(i) * K + k) * C + c, valid, m[i]);
		CT out[R * R][V];
		sandwich<M, R, 4, R, t, CT, V>(m, out);
#pragma unroll
		for (int i = 0; i < R * R; i++)
		{
			T *dst = dw + (k * R * R + i) * C + c;
			CT o[V];
#pragma unroll
			for (int v = 0; v < V; v++)
				o[v] = alpha * out[i][v];
			if (beta != static_cast<CT>(0))
			{
				CT old[V];
				load_vec<T, V, CT>(dst, valid, old);
#pragma unroll
				for (int v = 0; v < V; v++)
					o[v] += beta * old[v];
			}
			store_vec<T, V>(dst, valid, o);
		}
	}

	/* Channels per work-item: as many as 16 bytes of the wider of the two types hold, but never so many that the t x t tile
	 * (t*t values per channel, twice during the products) pushes the kernel to one or two wavefronts per SIMD: these kernels
	 * live on many loads and stores in flight from many wavefronts. */
#ifndef AVHIP_WINOGRAD_WIDTH_T6
#  define AVHIP_WINOGRAD_WIDTH_T6 2
#endif
#ifndef AVHIP_WINOGRAD_WIDTH_T4
#  define AVHIP_WINOGRAD_WIDTH_T4 4
#endif
	template<int M, int R, typename T, typename TM> struct VecOf
	{
		static constexpr int wider = sizeof(T) > sizeof(TM) ? sizeof(T) : sizeof(TM);
		static constexpr int wide = 4 * sizeof(float) / wider;
		static constexpr int cap = (M + R - 1 >= 6) ? AVHIP_WINOGRAD_WIDTH_T6 : AVHIP_WINOGRAD_WIDTH_T4;
		static constexpr int value = wide > cap ? cap : wide;
	};
	/* The width to launch with: VecOf's when every access of a [.., C] tensor stays aligned to it, else 1. */
	template<int M, int R, typename T, typename TM>
	int pick_vec(int C, const void *p0, const void *p1, const void *p2 = nullptr)
	{
		constexpr int VV = VecOf<M, R, T, TM>::value;
		const size_t need = VV * VecOf<M, R, T, TM>::wider;
		if (VV > 1 && C % VV == 0 && aligned_to(p0, need) && aligned_to(p1, need) && (p2 == nullptr || aligned_to(p2, need)))
			return VV;
		return 1;
	}

	template<typename T> typename Traits<T>::compute host_scalar(const void *p)
	{
		if (p == nullptr)
			return static_cast<typename Traits<T>::compute>(0);
		return Traits<T>::load(*reinterpret_cast<const T*>(p));
	}

	template<int M, int R, typename T, typename TM>
	int launch_weight(hipStream_t s, const void *w, void *U, int K, int C, int invert)
	{
		const int V = pick_vec<M, R, T, TM>(C, w, U);
		const size_t items = static_cast<size_t>(K) * ((C + V - 1) / V);
		const dim3 grid(ceil_div(items, 256));
		if (V > 1)
			hipLaunchKernelGGL((k_weight_transform<M, R, T, TM, VecOf<M, R, T, TM>::value>), grid, dim3(256), 0, s, static_cast<const T*>(w), static_cast<TM*>(U), K, C,
					invert);
		else
			hipLaunchKernelGGL((k_weight_transform<M, R, T, TM, 1>), grid, dim3(256), 0, s, static_cast<const T*>(w), static_cast<TM*>(U), K, C, invert);
		return 0;
	}
	template<int M, int R, typename T, typename TM>
	int launch_input(hipStream_t s, const void *x, void *Vm, int N, int H, int W, int C, int pad_h, int pad_w, const void *padding_value)
	{
		const int Th = (H + M - 1) / M, Tw = (W + M - 1) / M;
		const int V = pick_vec<M, R, T, TM>(C, x, Vm);
		const size_t items = static_cast<size_t>(N) * Th * Tw * ((C + V - 1) / V);
		const dim3 grid(ceil_div(items, 256));
		const typename Traits<T>::compute padv = host_scalar<T>(padding_value);
		const bool narrow = items < (1ull << 31) && static_cast<uint64_t>(H) * W * C < (1ull << 31);
#define AVHIP_LAUNCH_INPUT(WIDTH, IDX) hipLaunchKernelGGL((k_input_transform<M, R, T, TM, WIDTH, IDX>), grid, dim3(256), 0, s, static_cast<const T*>(x), \
		static_cast<TM*>(Vm), N, H, W, C, Th, Tw, pad_h, pad_w, padv)
		const bool buffered = padv == static_cast<typename Traits<T>::compute>(0) && static_cast<uint64_t>(N) * H * W * C * sizeof(T) < (1ull << 31);
		if (V > 1 && narrow && buffered)
		{
			constexpr int WIDTH = VecOf<M, R, T, TM>::value;
			if constexpr (WIDTH > 1 && (sizeof(T) * WIDTH == 4 || sizeof(T) * WIDTH == 8 || sizeof(T) * WIDTH == 16))
				hipLaunchKernelGGL((k_input_transform<M, R, T, TM, WIDTH, uint32_t, true>), grid, dim3(256), 0, s, static_cast<const T*>(x), static_cast<TM*>(Vm), N, H, W,
						C, Th, Tw, pad_h, pad_w, padv);
			else
				AVHIP_LAUNCH_INPUT(WIDTH, uint32_t);
		}
		else if (V > 1 && narrow)
			AVHIP_LAUNCH_INPUT((VecOf<M, R, T, TM>::value), uint32_t);
		else if (V > 1)
			AVHIP_LAUNCH_INPUT((VecOf<M, R, T, TM>::value), size_t);
		else if (narrow)
			AVHIP_LAUNCH_INPUT(1, uint32_t);
		else
			AVHIP_LAUNCH_INPUT(1, size_t);
#undef AVHIP_LAUNCH_INPUT
		return 0;
	}
	template<int M, int R, typename T, typename TM>
	int launch_output(hipStream_t s, const void *Mx, void *y, const void *bias, const void *z, int N, int H, int W, int K, double alpha1, double alpha2,
			double beta, int activation)
	{
		typedef typename Traits<T>::compute CT;
		const int Th = (H + M - 1) / M, Tw = (W + M - 1) / M;
		int V = pick_vec<M, R, T, TM>(K, Mx, y, z);
		const size_t items = static_cast<size_t>(N) * Th * Tw * ((K + V - 1) / V);
		const dim3 grid(ceil_div(items, 256));
#define AVHIP_LAUNCH_OUTPUT(WIDTH, ACT, IDX) hipLaunchKernelGGL((k_output_transform<M, R, T, TM, WIDTH, ACT, IDX>), grid, dim3(256), 0, s, \
		static_cast<const TM*>(Mx), static_cast<T*>(y), static_cast<const CT*>(bias), static_cast<const T*>(z), N, H, W, K, Th, Tw, static_cast<CT>(alpha1), \
		static_cast<CT>(alpha2), static_cast<CT>(beta), activation)
		/* LINEAR / RELU get their own instance: a nine-way switch per element makes the compiler evaluate every function */
		const bool simple = is_simple_activation(activation);
		const bool narrow = items < (1ull << 31) && static_cast<uint64_t>(H) * W < (1ull << 31);
		/* 16-bit matrices and tensors, t = 4, a problem of at most one round of resident workgroups (8 of 256 work-items on each
		 * of 256 compute units): 8 channels per work-item, i.e. 16-byte loads and stores.  A kernel this short is paced by how
		 * fast its accesses go out, not by how many wavefronts overlap (config 2, fp16 M: 22 -> 17.5 us); over several rounds
		 * the narrower work-items win by a few per cent, and the input transform is slower with 8 at every size. */
		constexpr int WIDE = VecOf<M, R, T, TM>::wide;
		if constexpr (WIDE == 8 && VecOf<M, R, T, TM>::value == 4 && M + R - 1 == 4)
		{
			if (V > 1 && simple && narrow && K % WIDE == 0 && items <= 256u * 8u * 256u && aligned_to(Mx, 16) && aligned_to(y, 16) && (z == nullptr || aligned_to(z, 16)))
			{
				const dim3 wide_grid(ceil_div(items / 2, 256));
				hipLaunchKernelGGL((k_output_transform<M, R, T, TM, WIDE, ACT_SIMPLE, uint32_t>), wide_grid, dim3(256), 0, s, static_cast<const TM*>(Mx), static_cast<T*>(y),
						static_cast<const CT*>(bias), static_cast<const T*>(z), N, H, W, K, Th, Tw, static_cast<CT>(alpha1), static_cast<CT>(alpha2), static_cast<CT>(beta),
						activation);
				return 0;
			}
		}
		if (V > 1 && simple && narrow)
			AVHIP_LAUNCH_OUTPUT((VecOf<M, R, T, TM>::value), ACT_SIMPLE, uint32_t);
		else if (V > 1 && narrow)
			AVHIP_LAUNCH_OUTPUT((VecOf<M, R, T, TM>::value), ACT_ANY, uint32_t);
		else if (V > 1)
			AVHIP_LAUNCH_OUTPUT((VecOf<M, R, T, TM>::value), ACT_ANY, size_t);
		else if (narrow)
			AVHIP_LAUNCH_OUTPUT(1, ACT_ANY, uint32_t);
		else
			AVHIP_LAUNCH_OUTPUT(1, ACT_ANY, size_t);
#undef AVHIP_LAUNCH_OUTPUT
		return 0;
	}

	template<int M, int R, typename T, typename TM>
	int launch_gradient(hipStream_t s, const void *dy, void *Mx, int N, int H, int W, int K)
	{
		const int Th = (H + M - 1) / M, Tw = (W + M - 1) / M;
		const int V = pick_vec<M, R, T, TM>(K, dy, Mx);
		const size_t items = static_cast<size_t>(N) * Th * Tw * ((K + V - 1) / V);
		const dim3 grid(ceil_div(items, 256));
		if (V > 1)
			hipLaunchKernelGGL((k_gradient_transform<M, R, T, TM, VecOf<M, R, T, TM>::value>), grid, dim3(256), 0, s, static_cast<const T*>(dy),
					static_cast<TM*>(Mx), N, H, W, K, Th, Tw);
		else
			hipLaunchKernelGGL((k_gradient_transform<M, R, T, TM, 1>), grid, dim3(256), 0, s, static_cast<const T*>(dy), static_cast<TM*>(Mx), N, H, W, K, Th,
					Tw);
		return 0;
	}
	template<int M, int R, typename T, typename TM>
	int launch_update(hipStream_t s, const void *Mx, void *dw, int K, int C, double alpha, double beta)
	{
		typedef typename Traits<T>::compute CT;
		const int V = pick_vec<M, R, T, TM>(C, Mx, dw);
		const size_t items = static_cast<size_t>(K) * ((C + V - 1) / V);
		const dim3 grid(ceil_div(items, 256));
		if (V > 1)
			hipLaunchKernelGGL((k_update_transform<M, R, T, TM, VecOf<M, R, T, TM>::value>), grid, dim3(256), 0, s, static_cast<const TM*>(Mx),
					static_cast<T*>(dw), K, C, static_cast<CT>(alpha), static_cast<CT>(beta));
		else
			hipLaunchKernelGGL((k_update_transform<M, R, T, TM, 1>), grid, dim3(256), 0, s, static_cast<const TM*>(Mx), static_cast<T*>(dw), K, C,
					static_cast<CT>(alpha), static_cast<CT>(beta));
		return 0;
	}

	/* Supported (tensor dtype, matrix dtype) pairs: equal types (the reference's behaviour), and fp16 or fp32 matrices
	 * for 16-bit tensors.  CALL is instantiated with <T, TM>. */
#define AVHIP_DISPATCH_PAIR(dtype, mat_dtype, CALL)                                              \
	switch (dtype)                                                                                 \
	{                                                                                              \
		case DT_FLOAT32:                                                                           \
			if (mat_dtype == DT_FLOAT32) { CALL(float, float); }                                   \
			return AVHIP_UNSUPPORTED_DATATYPE;                                                     \
		case DT_FLOAT64:                                                                           \
			if (mat_dtype == DT_FLOAT64) { CALL(double, double); }                                 \
			return AVHIP_UNSUPPORTED_DATATYPE;                                                     \
		case DT_FLOAT16:                                                                           \
			if (mat_dtype == DT_FLOAT16) { CALL(f16_t, f16_t); }                                   \
			if (mat_dtype == DT_FLOAT32) { CALL(f16_t, float); }                                   \
			return AVHIP_UNSUPPORTED_DATATYPE;                                                     \
		case DT_BFLOAT16:                                                                          \
			if (mat_dtype == DT_BFLOAT16) { CALL(bf16_t, bf16_t); }                                \
			if (mat_dtype == DT_FLOAT16) { CALL(bf16_t, f16_t); }                                  \
			if (mat_dtype == DT_FLOAT32) { CALL(bf16_t, float); }                                  \
			return AVHIP_UNSUPPORTED_DATATYPE;                                                     \
		default:                                                                                   \
			return AVHIP_UNSUPPORTED_DATATYPE;                                                     \
	}

#define AVHIP_DISPATCH_MR(m, r, FN, T, TM, ...)                                                  \
	if (m == 2 && r == 3) return FN<2, 3, T, TM>(__VA_ARGS__);                                    \
	if (m == 4 && r == 3) return FN<4, 3, T, TM>(__VA_ARGS__);                                    \
	if (m == 2 && r == 5) return FN<2, 5, T, TM>(__VA_ARGS__);                                    \
	return AVHIP_NOT_SUPPORTED;
}

extern "C"
{
	int avhip_winograd_weight_transform(void *stream, int dtype, int mat_dtype, int m, int r, int invert, const void *w, void *U, int K, int C)
	{
		if (w == nullptr || U == nullptr || K <= 0 || C <= 0)
			return AVHIP_BAD_PARAM;
		hipStream_t s = static_cast<hipStream_t>(stream);
#define CALL(T, TM) AVHIP_DISPATCH_MR(m, r, launch_weight, T, TM, s, w, U, K, C, invert)
		AVHIP_DISPATCH_PAIR(dtype, mat_dtype, CALL)
#undef CALL
	}

	int avhip_winograd_input_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *x, void *V, int N, int H, int W, int C,
			int pad_h, int pad_w, const void *padding_value)
	{
		if (x == nullptr || V == nullptr || N <= 0 || H <= 0 || W <= 0 || C <= 0)
			return AVHIP_BAD_PARAM;
		hipStream_t s = static_cast<hipStream_t>(stream);
#define CALL(T, TM) AVHIP_DISPATCH_MR(m, r, launch_input, T, TM, s, x, V, N, H, W, C, pad_h, pad_w, padding_value)
		AVHIP_DISPATCH_PAIR(dtype, mat_dtype, CALL)
#undef CALL
	}

	int avhip_winograd_output_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *M, void *y, const void *bias, const void *z,
			int N, int H, int W, int K, double alpha1, double alpha2, double beta, int activation)
	{
		if (M == nullptr || y == nullptr || N <= 0 || H <= 0 || W <= 0 || K <= 0)
			return AVHIP_BAD_PARAM;
		hipStream_t s = static_cast<hipStream_t>(stream);
#define CALL(T, TM) AVHIP_DISPATCH_MR(m, r, launch_output, T, TM, s, M, y, bias, z, N, H, W, K, alpha1, alpha2, beta, activation)
		AVHIP_DISPATCH_PAIR(dtype, mat_dtype, CALL)
#undef CALL
	}

	int avhip_winograd_gradient_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *dy, void *M, int N, int H, int W, int K)
	{
		if (dy == nullptr || M == nullptr || N <= 0 || H <= 0 || W <= 0 || K <= 0)
			return AVHIP_BAD_PARAM;
		hipStream_t s = static_cast<hipStream_t>(stream);
#define CALL(T, TM) AVHIP_DISPATCH_MR(m, r, launch_gradient, T, TM, s, dy, M, N, H, W, K)
		AVHIP_DISPATCH_PAIR(dtype, mat_dtype, CALL)
#undef CALL
	}

	int avhip_winograd_update_transform(void *stream, int dtype, int mat_dtype, int m, int r, const void *M, void *dw, int K, int C, double alpha,
			double beta)
	{
		if (M == nullptr || dw == nullptr || K <= 0 || C <= 0)
			return AVHIP_BAD_PARAM;
		hipStream_t s = static_cast<hipStream_t>(stream);
#define CALL(T, TM) AVHIP_DISPATCH_MR(m, r, launch_update, T, TM, s, M, dw, K, C, alpha, beta)
		AVHIP_DISPATCH_PAIR(dtype, mat_dtype, CALL)
#undef CALL
	}
}
