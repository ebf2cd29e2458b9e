/*
 * conv_thin.hpp -- internal interface of the kernel for convolutions over few input channels with filters of any size
 * (conv_thin.hip).
 */
#ifndef AVHIP_CONV_THIN_HPP_
#define AVHIP_CONV_THIN_HPP_

#include "conv_epilogue.hpp"

namespace avhip
{
	/* Launches the kernel that keeps an image tile in LDS and gathers the MFMA operand from it piece by piece when a pixel of
	 * x is at most 64 bytes, a filter row of w (R * S * C elements) at most 1024 bytes and tile, filters and tables fit LDS,
	 * and returns true; returns false without side effects otherwise.  Any stride, dilation and mode.  The caller has
	 * established: zero padding value, LINEAR or RELU activation, tensors below 2 GiB. */
	template<typename TE, typename Epi>
	bool conv_thin_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi);
}

#endif /* AVHIP_CONV_THIN_HPP_ */
