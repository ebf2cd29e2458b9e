/*
 * conv_stem.hpp -- internal interface of the kernel for convolutions over very few input channels (conv_stem.hip).
 */
#ifndef AVHIP_CONV_STEM_HPP_
#define AVHIP_CONV_STEM_HPP_

#include "conv_epilogue.hpp"

namespace avhip
{
	/* Launches the register-operand kernel when a pixel of x is exactly 8 bytes (4 channels of a 16-bit type, 8 of int8) and
	 * the filter has at most 12 taps, and returns true; returns false without side effects otherwise.  The caller has
	 * established: zero padding value, LINEAR or RELU activation, tensors below 2 GiB. */
	template<typename TE, typename Epi>
	bool conv_stem_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi);
}

#endif /* AVHIP_CONV_STEM_HPP_ */
