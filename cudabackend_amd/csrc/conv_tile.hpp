/*
 * conv_tile.hpp -- internal interface of the image-tile implicit-GEMM kernel (conv_tile.hip).
 */
#ifndef AVHIP_CONV_TILE_HPP_
#define AVHIP_CONV_TILE_HPP_

#include "conv_epilogue.hpp"

namespace avhip
{
	/* Launches the tile kernel when the problem suits it (stride 1, dilation 1, a tile of the image with its halo fits
	 * in LDS) and returns true; returns false without side effects otherwise.  The caller has already established the
	 * fast-path conditions: 16-byte aligned tensors below 2 GiB, channel count a multiple of the 16-byte chunk, zero
	 * padding value, LINEAR or RELU activation. */
	template<typename TE, typename Epi>
	bool conv_tile_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi);
}

#endif /* AVHIP_CONV_TILE_HPP_ */
