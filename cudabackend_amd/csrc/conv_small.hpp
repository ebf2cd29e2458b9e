/*
 * conv_small.hpp -- internal interface of the small-problem implicit-GEMM kernel (conv_small.hip).
 */
#ifndef AVHIP_CONV_SMALL_HPP_
#define AVHIP_CONV_SMALL_HPP_

#include "conv_epilogue.hpp"

namespace avhip
{
	/* Launches the one-wavefront-per-tile kernel and returns true when the problem is so small that the 128 x 128 (or
	 * 256 x 64) workgroup tiles of the other kernels would occupy less than `busy_workgroups` workgroups; returns false
	 * without side effects otherwise.  The caller has established the fast-path conditions (16-byte aligned tensors below
	 * 2 GiB, channel count a multiple of the 16-byte chunk, zero padding value, LINEAR or RELU, vector stores allowed). */
	template<typename TE, typename Epi>
	bool conv_small_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi, int64_t big_tile_workgroups);

	/* The launcher's estimates, in microseconds, for a layer with elements of `element_bytes`: what the one-wavefront-per-tile
	 * kernel would take, and what a kernel with 128 x 128 workgroup tiles would take for `big_tile_workgroups` of them. */
	struct SmallProblemEstimate
	{
		double small_us, workgroup_tiles_us;
		bool split_k; /* four wavefronts share a tile's k range */
	};
	SmallProblemEstimate conv_small_estimate(const avhipConvShape &s, int element_bytes, int64_t big_tile_workgroups);
	/* Whether the launcher would send the layer to that kernel (the threshold of avhip_set_small_problem_threshold and the
	 * two estimates), given that the kernel can run it. */
	bool conv_small_preferred(const avhipConvShape &s, int element_bytes, int64_t big_tile_workgroups);
}

#endif /* AVHIP_CONV_SMALL_HPP_ */
