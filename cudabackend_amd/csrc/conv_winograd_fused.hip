/*
 * conv_winograd_fused.hip -- single-kernel Winograd F(2x2, 3x3) convolution (placeholder until the kernel lands).
 */
#include "common.hpp"

extern "C" int avhip_conv2d_winograd_fused(void *stream, int dtype, const avhipConvShape *shape, const void *x, const void *U, const void *bias,
		const void *z, void *y, double alpha1, double alpha2, double beta, int activation)
{
	(void) stream; (void) dtype; (void) shape; (void) x; (void) U; (void) bias; (void) z; (void) y; (void) alpha1; (void) alpha2; (void) beta; (void) activation;
	return AVHIP_NOT_SUPPORTED;
}
