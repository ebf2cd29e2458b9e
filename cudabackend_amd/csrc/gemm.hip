/*
 * gemm.hip -- C[b] = alpha * op(A[b]) op(B[b]) + beta * C[b] for row-major operands.
 *
 * Replaces the cuBLAS calls behind cudaGemm / cudaGemmBatched of the reference (src/gemm.cpp:25-209).  The batched
 * (N, T) form  M[b] = V[b] * U[b]^T  is the matrix-core stage of non-fused Winograd (app/CudaBackend.cu:417-418): both
 * operands are contiguous along k, so it runs on the shared MFMA engine with fp32 (int32 for int8) accumulation and the
 * result is rounded once, to nearest even, on store.  Every other operand form, and fp64, goes through a small LDS-tiled
 * kernel that exists for completeness of the API, not for speed.
 * Unlike the reference there is a bf16 case, fp16 always accumulates in fp32, and the result of a 16-bit product may be
 * kept in fp32.
 */
#include <type_traits>

#include "mfma_core.hpp"
#include "persistent_gemm.hpp"
#include "resident_gemm.hpp"

namespace
{
	using namespace avhip;

	/* Operand rows of a plain row-major matrix: row r starts at base + r * ld, k runs along the row.
	 * General form: any alignment, any K; partial chunks are assembled element by element. */
	template<typename TE, bool FAST>
	struct RowLoader
	{
		const TE *rows[FETCH_PASSES]; /* start of this work-item's rows, nullptr outside the matrix */
		int K, k;
		bool vec_ok;
		__device__ inline RowLoader(const TE *base, int nrows, int K_, int ld, int row0, bool vec_ok_) :
				K(K_), k(0), vec_ok(vec_ok_)
		{
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int row = row0 + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
				rows[q] = row < nrows ? base + static_cast<size_t>(row) * ld : nullptr;
			}
		}
		__device__ inline uint4 load(int q, int part) const
		{
			constexpr int E = 16 / sizeof(TE);
			if (rows[q] == nullptr)
				return make_uint4(0u, 0u, 0u, 0u);
			const int kk = k + part * E;
			return fetch_chunk<TE>(rows[q] + kk, K - kk, vec_ok);
		}
		__device__ inline void next()
		{
			k += STEP_BYTES / sizeof(TE);
		}
	};
	/* Fast form: rows 16-byte aligned, K a multiple of the chunk, matrix below 2 GiB: branch-free buffer loads. */
	template<typename TE>
	struct RowLoader<TE, true>
	{
		__amdgpu_buffer_rsrc_t rsrc;
		unsigned int origin[FETCH_PASSES]; /* byte offset of this work-item's chunk in its rows; OUT_OF_RANGE stays out of range */
		unsigned int chunk_bytes, k_bytes, K_bytes;
		__device__ inline RowLoader(const TE *base, int nrows, int K, int ld, int row0, bool) :
				k_bytes(0), K_bytes(K * sizeof(TE))
		{
			rsrc = make_buffer(base, (static_cast<unsigned int>(nrows - 1) * ld + K) * sizeof(TE));
			chunk_bytes = (threadIdx.x % STEP_CHUNKS) * 16;
#pragma unroll
			for (int q = 0; q < FETCH_PASSES; q++)
			{
				const int row = row0 + threadIdx.x / STEP_CHUNKS + FETCH_ROWS * q;
				origin[q] = row < nrows ? static_cast<unsigned int>(row) * ld * sizeof(TE) + chunk_bytes : OUT_OF_RANGE;
			}
		}
		__device__ inline uint4 load(int q, int) const
		{
			return buffer_fetch(rsrc, (k_bytes + chunk_bytes < K_bytes) ? origin[q] + k_bytes : OUT_OF_RANGE);
		}
		__device__ inline void next()
		{
			k_bytes += STEP_BYTES;
		}
	};

	/* Writes alpha * acc + beta * C for 4 consecutive columns (fewer at the right edge of the matrix). */
	template<typename TC>
	__device__ inline void store_c(TC *p, int valid, bool vec, const float (&acc)[4], float alpha, float beta)
	{
		float v[4];
#pragma unroll
		for (int q = 0; q < 4; q++)
			v[q] = alpha * acc[q];
		if (beta != 0.0f)
		{
			float old[4];
			load_vec<TC, 4, float>(p, valid, old, vec);
#pragma unroll
			for (int q = 0; q < 4; q++)
				v[q] += beta * old[q];
		}
		store_vec<TC, 4, float, true>(p, valid, v, vec); /* streaming: C is not read back by this kernel */
	}
	__device__ inline void store_c(int *p, int valid, bool vec, const int (&acc)[4], int alpha, int beta)
	{
		int v[4];
#pragma unroll
		for (int q = 0; q < 4; q++)
		{
			v[q] = alpha * acc[q];
			if (beta != 0 && q < valid)
				v[q] += beta * p[q];
		}
		if (vec && valid >= 4)
			*reinterpret_cast<int4*>(p) = make_int4(v[0], v[1], v[2], v[3]);
		else
		{
#pragma unroll
			for (int q = 0; q < 4; q++)
				if (q < valid)
					p[q] = v[q];
		}
	}

	template<typename TE, typename TC, bool FAST>
	__global__ __launch_bounds__(256, 2) void k_gemm_nt_mfma(const TE *__restrict__ A, const TE *__restrict__ B, TC *C, int M, int N, int K, int lda, int ldb,
			int ldc, int64_t strideA, int64_t strideB, int64_t strideC, typename Mma<TE>::scalar_t alpha, typename Mma<TE>::scalar_t beta, int vec_ok)
	{
		__shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];
		constexpr int KE = STEP_BYTES / sizeof(TE);
		const int batch = blockIdx.z;
		unsigned int row_block, column_block;
		xcd_tile(row_block, column_block); /* the column blocks of a row block share A through one L2 */
		const int m0 = row_block * BLOCK_M;
		const int n0 = column_block * BLOCK_N;

		RowLoader<TE, FAST> la(A + batch * strideA, M, K, lda, m0, (vec_ok & 1) != 0);
		RowLoader<TE, FAST> lb(B + batch * strideB, N, K, ldb, n0, (vec_ok & 1) != 0);
		typename Mma<TE>::acc_t acc[2][2];
		block_mma<TE>(lds, (K + KE - 1) / KE, la, lb, acc);

		TC *c = C + batch * strideC;
		const bool vec_c = (vec_ok & 2) != 0;
		const int cc = n0 + drain_column<2>();
		drain_tile<TE, 2, 2>(lds, acc, [&](int r, const typename Mma<TE>::scalar_t (&v)[4], int) __attribute__((always_inline))
		{
			const int row = m0 + r;
			if (row < M && cc < N)
				store_c(c + static_cast<size_t>(row) * ldc + cc, N - cc, vec_c, v, alpha, beta);
		});
	}

	/* C = alpha * acc + beta * C as the epilogue of the persistent short-k product (floating types). */
	template<typename TC>
	struct GemmEpilogue
	{
		typedef float scalar_t;
		static constexpr int wide = sizeof(TC) >= 4 ? 4 : 8; /* one 16-byte store */
		template<int W> struct ColumnsT
		{
		};
		template<int W> struct Residual /* C has no residual term */
		{
		};
		TC *c;
		float alpha, beta;
		__device__ __forceinline__ void pin()
		{
			keep_in_sgpr(alpha);
			keep_in_sgpr(beta);
		}
		__device__ __forceinline__ void load_columns(int, ColumnsT<1>&) const
		{
		}
		template<int W>
		__device__ static __forceinline__ void pick_columns(const ColumnsT<1>*, int, ColumnsT<W>&)
		{
		}
		template<int ACT, bool VEC, int W>
		__device__ __forceinline__ void store_at(int64_t idx, int, const float (&v)[W], const ColumnsT<W>&) const
		{
			float t[W];
#pragma unroll
			for (int q = 0; q < W; q++)
				t[q] = alpha * v[q];
			if (beta != 0.0f)
			{
				float old[W];
				load_vec<TC, W, float>(c + idx, W, old, true);
#pragma unroll
				for (int q = 0; q < W; q++)
					t[q] += beta * old[q];
			}
			store_vec<TC, W, float, true>(c + idx, W, t, true); /* streaming: C is not read back by this kernel */
		}
		static constexpr bool masked_stores = true;
		static constexpr bool residual_ahead = false;
		static constexpr int out_bytes = sizeof(TC);
		__device__ __forceinline__ char *out() const { return reinterpret_cast<char*>(c); }
		template<int W, typename Sink>
		__device__ __forceinline__ void store_masked(bool exists, int64_t idx, int, const float (&v)[W], const ColumnsT<W>&, const Sink &sink) const
		{
			static_assert(W * sizeof(TC) == 16, "one 16-byte run");
			float t[W];
#pragma unroll
			for (int q = 0; q < W; q++)
				t[q] = alpha * v[q];
			if (beta != 0.0f && exists)
			{
				float old[W];
				load_vec<TC, W, float>(c + idx, W, old, true);
#pragma unroll
				for (int q = 0; q < W; q++)
					t[q] += beta * old[q];
			}
			typedef unsigned int words_t __attribute__((ext_vector_type(4)));
			union
			{
				Pack<TC, W> p;
				words_t words;
			} u;
#pragma unroll
			for (int q = 0; q < W; q++)
				u.p.v[q] = Traits<TC>::store(t[q]);
			sink(u.words);
		}
	};

	template<typename TE, typename TC, int STEPS, int TM>
	__global__ __launch_bounds__(256, 2) void k_gemm_nt_persistent(const TE *__restrict__ A, const TE *__restrict__ B, PersistentGeom g, GemmEpilogue<TC> epi)
	{
		__shared__ __attribute__((aligned(16))) char lds[PERSISTENT_LDS_BYTES];
		persistent_nt_gemm<TE, GemmEpilogue<TC>, STEPS, TM>(lds, A, B, g, epi);
	}

	template<typename TE, typename TC, int STEPS>
	__global__ __launch_bounds__(256, RESIDENT_OCCUPANCY) void k_gemm_nt_resident(const TE *__restrict__ A, const TE *__restrict__ B, ResidentGeom g, GemmEpilogue<TC> epi)
	{
		__shared__ __attribute__((aligned(16))) char lds[RESIDENT_LDS_BYTES];
		resident_nt_gemm<TE, GemmEpilogue<TC>, STEPS>(lds, A, B, g, epi);
	}

	/* Any operand form, any supported type: 16 x 16 outputs per workgroup, k in slices of 16 through LDS. */
	template<typename TA, typename TC, typename CT>
	__global__ __launch_bounds__(256) void k_gemm_generic(const TA *__restrict__ A, const TA *__restrict__ B, TC *C, int M, int N, int K, int opA, int opB,
			int lda, int ldb, int ldc, int64_t strideA, int64_t strideB, int64_t strideC, CT alpha, CT beta)
	{
		__shared__ CT sa[16][17];
		__shared__ CT sb[16][17];
		const int batch = blockIdx.z;
		const TA *a = A + batch * strideA;
		const TA *b = B + batch * strideB;
		const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
		const int row = blockIdx.y * 16 + ty;
		const int col = blockIdx.x * 16 + tx;
		CT acc = 0;
		for (int k0 = 0; k0 < K; k0 += 16)
		{
			{ // sa[ty][tx] = opA(A)[row0 + ty][k0 + tx]
				const int r = blockIdx.y * 16 + ty, k = k0 + tx;
				CT v = 0;
				if (r < M && k < K)
					v = static_cast<CT>(opA ? a[static_cast<size_t>(k) * lda + r] : a[static_cast<size_t>(r) * lda + k]);
				sa[ty][tx] = v;
			}
			{ // sb[ty][tx] = opB(B)[k0 + ty][col0 + tx]
				const int k = k0 + ty, cidx = blockIdx.x * 16 + tx;
				CT v = 0;
				if (k < K && cidx < N)
					v = static_cast<CT>(opB ? b[static_cast<size_t>(cidx) * ldb + k] : b[static_cast<size_t>(k) * ldb + cidx]);
				sb[ty][tx] = v;
			}
			__syncthreads();
#pragma unroll
			for (int k = 0; k < 16; k++)
				acc += sa[ty][k] * sb[k][tx];
			__syncthreads();
		}
		if (row < M && col < N)
		{
			TC *p = C + batch * strideC + static_cast<size_t>(row) * ldc + col;
			CT v = alpha * acc;
			if (beta != static_cast<CT>(0))
				v += beta * static_cast<CT>(*p);
			*p = static_cast<TC>(v);
		}
	}

	/* Thin value wrappers so that the generic kernel can static_cast 16-bit storage types. */
	struct bf16_val
	{
		bf16_t raw;
		__device__ operator float() const { return bf16_to_float(raw); }
		__device__ bf16_val() = default;
		__device__ bf16_val(float f) : raw(float_to_bf16(f)) {}
	};

	template<typename TE, typename TC>
	bool launch_persistent(hipStream_t s, const void *A, const void *B, void *C, int batch, int M, int N, int K, int lda, int ldb, int ldc, int64_t sA,
			int64_t sB, int64_t sC, double alpha, double beta, bool fast)
	{
		if constexpr (std::is_same<typename Mma<TE>::scalar_t, float>::value)
		{
			typedef GemmEpilogue<TC> Epi;
			const int64_t row_bytes = static_cast<int64_t>(K) * sizeof(TE);
			const int steps = static_cast<int>((row_bytes + STEP_BYTES - 1) / STEP_BYTES);
			if (!fast || steps > PERSISTENT_MAX_STEPS)
				return false;
			/* fp32 products are bound by the matrix cores (sixteen-pass MFMAs), not by operand traffic: half-height tiles cost
			 * them nothing and split the work into rounds more evenly (the Winograd layer measured: 1152 tiles of 128 rows are
			 * 2.25 rounds of the 512 resident workgroups, 2304 of 64 rows are 4.5) */
			constexpr int TM = sizeof(TE) >= 4 ? 1 : 2;
			constexpr int ROWS = 64 * TM;
			/* whole 16-byte runs of C, rows of C a multiple of them apart */
			if (N % Epi::wide != 0 || ldc % Epi::wide != 0 || sC % Epi::wide != 0 || !aligned_to(C, 16) || ldc >= (1 << 22))
				return false;
			const int64_t a_bytes = ((batch - 1) * sA + static_cast<int64_t>(M - 1) * lda + K) * static_cast<int64_t>(sizeof(TE));
			const int64_t b_bytes = ((batch - 1) * sB + static_cast<int64_t>(N - 1) * ldb + K) * static_cast<int64_t>(sizeof(TE));
			const int64_t row_blocks = ceil_div(M, ROWS), col_blocks = ceil_div(N, BLOCK_N);
			const int64_t tiles = row_blocks * col_blocks * batch;
			if (sA < 0 || sB < 0 || a_bytes >= (1ll << 31) || b_bytes >= (1ll << 31) || tiles >= (1ll << 31) - 1024)
				return false;
			if (short_k_engine().load(std::memory_order_relaxed) == 0 && row_bytes % 16 == 0 && steps <= RESIDENT_MAX_STEPS)
			{
				ResidentGeom r;
				r.rows = M;
				r.cols = N;
				r.row_bytes = static_cast<unsigned int>(row_bytes);
				r.a_pitch = static_cast<unsigned int>(lda * sizeof(TE));
				r.b_pitch = static_cast<unsigned int>(ldb * sizeof(TE));
				r.a_batch = static_cast<unsigned int>(sA * sizeof(TE));
				r.b_batch = static_cast<unsigned int>(sB * sizeof(TE));
				r.a_bytes = static_cast<unsigned int>(a_bytes);
				r.b_bytes = static_cast<unsigned int>(b_bytes);
				r.c_batch = sC;
				r.c_pitch = ldc;
				r.table_columns = 0;
				const Epi epi { static_cast<TC*>(C), static_cast<float>(alpha), static_cast<float>(beta) };
				const dim3 grid(resident_plan(r, batch));
				const TE *ap = static_cast<const TE*>(A), *bp = static_cast<const TE*>(B);
				if (steps == 1)
					hipLaunchKernelGGL((k_gemm_nt_resident<TE, TC, 1>), grid, dim3(256), 0, s, ap, bp, r, epi);
				else if (steps == 2)
					hipLaunchKernelGGL((k_gemm_nt_resident<TE, TC, 2>), grid, dim3(256), 0, s, ap, bp, r, epi);
				else
					hipLaunchKernelGGL((k_gemm_nt_resident<TE, TC, 4>), grid, dim3(256), 0, s, ap, bp, r, epi);
				return true;
			}
			PersistentGeom g;
			g.rows = M;
			g.cols = N;
			g.row_bytes = static_cast<unsigned int>(row_bytes);
			g.a_pitch = static_cast<unsigned int>(lda * sizeof(TE));
			g.b_pitch = static_cast<unsigned int>(ldb * sizeof(TE));
			g.a_batch = static_cast<unsigned int>(sA * sizeof(TE));
			g.b_batch = static_cast<unsigned int>(sB * sizeof(TE));
			g.a_bytes = static_cast<unsigned int>(a_bytes);
			g.b_bytes = static_cast<unsigned int>(b_bytes);
			g.c_batch = sC;
			g.c_pitch = ldc;
			g.row_blocks = static_cast<int>(row_blocks);
			g.col_blocks = static_cast<int>(col_blocks);
			g.tiles = static_cast<int>(tiles);
			g.table_columns = 0;
			const Epi epi { static_cast<TC*>(C), static_cast<float>(alpha), static_cast<float>(beta) };
			const dim3 grid(persistent_workgroups(tiles));
			if (steps <= 2)
				hipLaunchKernelGGL((k_gemm_nt_persistent<TE, TC, 2, TM>), grid, dim3(256), 0, s, static_cast<const TE*>(A), static_cast<const TE*>(B), g, epi);
			else
				hipLaunchKernelGGL((k_gemm_nt_persistent<TE, TC, 4, TM>), grid, dim3(256), 0, s, static_cast<const TE*>(A), static_cast<const TE*>(B), g, epi);
			return true;
		}
		else
			return false;
	}

	template<typename TE, typename TC>
	int launch_mfma(hipStream_t s, const void *A, const void *B, void *C, int batch, int M, int N, int K, int lda, int ldb, int ldc, int64_t sA, int64_t sB,
			int64_t sC, double alpha, double beta)
	{
		typedef typename Mma<TE>::scalar_t S;
		const bool vec_ok = aligned_to(A, 16) && aligned_to(B, 16) && (lda * sizeof(TE)) % 16 == 0 && (ldb * sizeof(TE)) % 16 == 0
				&& (sA * sizeof(TE)) % 16 == 0 && (sB * sizeof(TE)) % 16 == 0;
		const bool vec_c = aligned_to(C, 4 * sizeof(TC)) && ldc % 4 == 0 && sC % 4 == 0;
		const dim3 grid(ceil_div(M, BLOCK_M), ceil_div(N, BLOCK_N), batch);
		const int flags = (vec_ok ? 1 : 0) | (vec_c ? 2 : 0);
		const bool small = (static_cast<int64_t>(M) * lda + K) * static_cast<int64_t>(sizeof(TE)) < (1ll << 31)
				&& (static_cast<int64_t>(N) * ldb + K) * static_cast<int64_t>(sizeof(TE)) < (1ll << 31);
		const bool fast = vec_ok && small && K % (16 / static_cast<int>(sizeof(TE))) == 0;
		/* a short k (the channel count of a Winograd layer): workgroups stay resident and pipeline across tiles */
		if (launch_persistent<TE, TC>(s, A, B, C, batch, M, N, K, lda, ldb, ldc, sA, sB, sC, alpha, beta, fast))
			return 0;
#define AVHIP_GEMM_ARGS static_cast<const TE*>(A), static_cast<const TE*>(B), static_cast<TC*>(C), M, N, K, lda, ldb, ldc, sA, sB, sC, static_cast<S>(alpha), \
		static_cast<S>(beta), flags
		if (fast)
			hipLaunchKernelGGL((k_gemm_nt_mfma<TE, TC, true>), grid, dim3(256), 0, s, AVHIP_GEMM_ARGS);
		else
			hipLaunchKernelGGL((k_gemm_nt_mfma<TE, TC, false>), grid, dim3(256), 0, s, AVHIP_GEMM_ARGS);
#undef AVHIP_GEMM_ARGS
		return 0;
	}
	template<typename TA, typename TC, typename CT>
	int launch_generic(hipStream_t s, const void *A, const void *B, void *C, int batch, int M, int N, int K, int opA, int opB, int lda, int ldb, int ldc,
			int64_t sA, int64_t sB, int64_t sC, double alpha, double beta)
	{
		const dim3 grid(ceil_div(N, 16), ceil_div(M, 16), batch);
		hipLaunchKernelGGL((k_gemm_generic<TA, TC, CT>), grid, dim3(256), 0, s, static_cast<const TA*>(A), static_cast<const TA*>(B), static_cast<TC*>(C), M, N,
				K, opA, opB, lda, ldb, ldc, sA, sB, sC, static_cast<CT>(alpha), static_cast<CT>(beta));
		return 0;
	}
}

namespace
{
	/* Eight independent accumulators per wavefront: enough MFMAs in flight to cover the pipeline depth without any memory
	 * access in the loop.  QUIET operands are almost all zero bits (the matrix cores toggle little and the clock stays near
	 * boost); otherwise every MFMA reads one of four A and two B register sets filled with hashed bits shaped into finite
	 * numbers of magnitude 0.5 .. 2, which is what the clock under a real workload's switching activity looks like. */
	template<typename TE> __device__ inline unsigned finite_bits(unsigned r);
	template<> __device__ inline unsigned finite_bits<f16_t>(unsigned r) { return (r & 0x83ff83ffu) | 0x38003800u; }
	template<> __device__ inline unsigned finite_bits<bf16_t>(unsigned r) { return (r & 0x80ff80ffu) | 0x3f003f00u; }
	template<> __device__ inline unsigned finite_bits<int8_t>(unsigned r) { return r; }
	template<> __device__ inline unsigned finite_bits<float>(unsigned r) { return (r & 0x80ffffffu) | 0x3f000000u; }
	__device__ inline unsigned hash_bits(unsigned v)
	{
		v ^= v >> 16;
		v *= 0x7feb352du;
		v ^= v >> 15;
		v *= 0x846ca68bu;
		v ^= v >> 16;
		return v;
	}
	template<typename TE, bool QUIET>
	__global__ __launch_bounds__(256) void k_mfma_rate_probe(int iterations, typename Mma<TE>::scalar_t *sink)
	{
		typename Mma<TE>::acc_t acc[8];
#pragma unroll
		for (int i = 0; i < 8; i++)
#pragma unroll
			for (int v = 0; v < 16; v++)
				acc[i][v] = 0;
		Chunk a[4], b[2];
#pragma unroll
		for (int i = 0; i < 4; i++)
		{
			if (QUIET)
				a[i].u = make_uint4(threadIdx.x, 0u, 0u, 0u);
			else
			{
				const unsigned seed = (blockIdx.x * 256u + threadIdx.x) * 32u + i * 4u;
				a[i].u = make_uint4(finite_bits<TE>(hash_bits(seed)), finite_bits<TE>(hash_bits(seed + 1)), finite_bits<TE>(hash_bits(seed + 2)),
						finite_bits<TE>(hash_bits(seed + 3)));
			}
		}
#pragma unroll
		for (int i = 0; i < 2; i++)
		{
			if (QUIET)
				b[i].u = make_uint4(0u, threadIdx.x & 1u, 0u, 0u);
			else
			{
				const unsigned seed = (blockIdx.x * 256u + threadIdx.x) * 32u + 16u + i * 4u;
				b[i].u = make_uint4(finite_bits<TE>(hash_bits(seed)), finite_bits<TE>(hash_bits(seed + 1)), finite_bits<TE>(hash_bits(seed + 2)),
						finite_bits<TE>(hash_bits(seed + 3)));
			}
		}
		for (int it = 0; it < iterations; it++)
		{
#pragma unroll
			for (int i = 0; i < 8; i++)
				Mma<TE>::run(a[i & 3], b[i >> 2], acc[i]);
		}
		typename Mma<TE>::scalar_t total = 0;
#pragma unroll
		for (int i = 0; i < 8; i++)
#pragma unroll
			for (int v = 0; v < 16; v++)
				total += acc[i][v];
		sink[static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x] = total;
	}
	template<typename TE>
	void launch_rate_probe(hipStream_t st, int workgroups, int iterations, int operands, void *sink)
	{
		typedef typename Mma<TE>::scalar_t scalar_t;
		if (operands == 0)
			hipLaunchKernelGGL((k_mfma_rate_probe<TE, true>), dim3(workgroups), dim3(256), 0, st, iterations, static_cast<scalar_t*>(sink));
		else
			hipLaunchKernelGGL((k_mfma_rate_probe<TE, false>), dim3(workgroups), dim3(256), 0, st, iterations, static_cast<scalar_t*>(sink));
	}
}

extern "C" int avhip_mfma_rate_probe(void *stream, int dtype, int workgroups, int iterations, int operands, void *sink)
{
	if (workgroups <= 0 || iterations <= 0 || sink == nullptr || operands < 0 || operands > 1)
		return AVHIP_BAD_PARAM;
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (dtype)
	{
		case DT_FLOAT16:
			launch_rate_probe<f16_t>(st, workgroups, iterations, operands, sink);
			return 0;
		case DT_BFLOAT16:
			launch_rate_probe<bf16_t>(st, workgroups, iterations, operands, sink);
			return 0;
		case DT_INT8:
			launch_rate_probe<int8_t>(st, workgroups, iterations, operands, sink);
			return 0;
		case DT_FLOAT32:
			/* Mma<float>::run issues four 32x32x2 MFMAs per call */
			launch_rate_probe<float>(st, workgroups, iterations, operands, sink);
			return 0;
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
}

extern "C" int avhip_gemm_batched(void *stream, int ab_dtype, int c_dtype, int opA, int opB, const void *A, const void *B, void *C, int batch, int M,
		int N, int K, int lda, int ldb, int ldc, int64_t strideA, int64_t strideB, int64_t strideC, double alpha, double beta)
{
	if (A == nullptr || B == nullptr || C == nullptr || batch <= 0 || M <= 0 || N <= 0 || K <= 0)
		return AVHIP_BAD_PARAM;
	if (batch > 65535)
		return AVHIP_NOT_SUPPORTED;
	hipStream_t s = static_cast<hipStream_t>(stream);
	const bool nt = (opA == 0 && opB != 0);
#define ARGS_MFMA s, A, B, C, batch, M, N, K, lda, ldb, ldc, strideA, strideB, strideC, alpha, beta
#define ARGS_GEN s, A, B, C, batch, M, N, K, opA, opB, lda, ldb, ldc, strideA, strideB, strideC, alpha, beta
	switch (ab_dtype)
	{
		case DT_FLOAT32:
			if (c_dtype != DT_FLOAT32)
				return AVHIP_UNSUPPORTED_DATATYPE;
			return nt ? launch_mfma<float, float>(ARGS_MFMA) : launch_generic<float, float, float>(ARGS_GEN);
		case DT_FLOAT64:
			if (c_dtype != DT_FLOAT64)
				return AVHIP_UNSUPPORTED_DATATYPE;
			return launch_generic<double, double, double>(ARGS_GEN);
		case DT_FLOAT16:
			if (c_dtype == DT_FLOAT16)
				return nt ? launch_mfma<f16_t, f16_t>(ARGS_MFMA) : launch_generic<f16_t, f16_t, float>(ARGS_GEN);
			if (c_dtype == DT_FLOAT32)
				return nt ? launch_mfma<f16_t, float>(ARGS_MFMA) : launch_generic<f16_t, float, float>(ARGS_GEN);
			return AVHIP_UNSUPPORTED_DATATYPE;
		case DT_BFLOAT16:
			if (c_dtype == DT_BFLOAT16)
				return nt ? launch_mfma<bf16_t, bf16_t>(ARGS_MFMA) : launch_generic<bf16_val, bf16_val, float>(ARGS_GEN);
			if (c_dtype == DT_FLOAT32)
				return nt ? launch_mfma<bf16_t, float>(ARGS_MFMA) : launch_generic<bf16_val, float, float>(ARGS_GEN);
			return AVHIP_UNSUPPORTED_DATATYPE;
		case DT_INT8:
			if (c_dtype != DT_INT32)
				return AVHIP_UNSUPPORTED_DATATYPE;
			return nt ? launch_mfma<int8_t, int>(ARGS_MFMA) : launch_generic<int8_t, int, int>(ARGS_GEN);
		default:
			return AVHIP_UNSUPPORTED_DATATYPE;
	}
#undef ARGS_MFMA
#undef ARGS_GEN
}
