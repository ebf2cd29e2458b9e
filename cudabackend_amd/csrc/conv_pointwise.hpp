/*
 * conv_pointwise.hpp -- internal interface of the persistent 1x1-convolution kernel (conv_pointwise.hip).
 */
#ifndef AVHIP_CONV_POINTWISE_HPP_
#define AVHIP_CONV_POINTWISE_HPP_

#include "conv_epilogue.hpp"

namespace avhip
{
	/* Launches the persistent kernel for a 1x1 filter with stride 1 and no padding and returns true; returns false without
	 * side effects when the problem is anything else or its output cannot be stored in whole 16-byte runs.  The caller has
	 * established the fast-path conditions: 16-byte aligned tensors below 2 GiB, channel count a multiple of the 16-byte
	 * chunk, LINEAR or RELU activation. */
	template<typename TE, typename Epi>
	bool conv_pointwise_launch(hipStream_t stream, const avhipConvShape &s, const void *x, const void *w, const Epi &epi);
}

#endif /* AVHIP_CONV_POINTWISE_HPP_ */
