/*
 * cpu_baseline.c  --  TEST / BENCH INFRASTRUCTURE ONLY.
 *
 * The CPU routines bench.py times next to the GPU numbers ("cpu_baseline", kind "port"): a plain
 * multi-threaded restatement of the direct convolution of app/CudaBackend.cu:122-201 with the
 * accumulation type of the path it stands beside (fp32, or int32 for int8).  They are never used as a
 * checker and never called by the product.  Built with -O3 -mavx2 -mfma -fopenmp.
 */
#include <stdint.h>
#include <stdlib.h>

/*
 * Timed CPU baseline (not a checker): fp32 NHWC direct convolution with fp32 accumulation,
 * zero padding, convolution mode, groups 1, bias + ReLU/linear epilogue, OpenMP over output rows.
 * The weights are re-laid as [R, S, C, K] once so that the innermost loop runs over contiguous
 * output channels and vectorises.  Returns 0, or -1 when the scratch allocation fails.
 */
int orc_conv2d_f32_omp(const float *x, const float *w, const float *bias, float *y, int N, int H, int W, int C, int K, int R, int S, int Ho, int Wo,
		int pad_h, int pad_w, int stride_h, int stride_w, int relu)
{
	float *wt = (float*) malloc(sizeof(float) * (size_t) R * S * C * K);
	if (wt == NULL)
		return -1;
	for (int k = 0; k < K; k++)
		for (int i = 0; i < R; i++)
			for (int j = 0; j < S; j++)
				for (int c = 0; c < C; c++)
					wt[(((size_t) i * S + j) * C + c) * K + k] = w[(((size_t) k * R + i) * S + j) * C + c];
#pragma omp parallel for collapse(2) schedule(static)
	for (int n = 0; n < N; n++)
		for (int oh = 0; oh < Ho; oh++)
		{
			float acc[1024];
			for (int ow = 0; ow < Wo; ow++)
			{
				float *yp = y + (((size_t) n * Ho + oh) * Wo + ow) * K;
				for (int k0 = 0; k0 < K; k0 += 1024)
				{
					const int kn = (K - k0) < 1024 ? (K - k0) : 1024;
					for (int k = 0; k < kn; k++)
						acc[k] = bias != NULL ? bias[k0 + k] : 0.0f;
					for (int i = 0; i < R; i++)
					{
						const int ih = pad_h + i + oh * stride_h;
						if (ih < 0 || ih >= H)
							continue;
						for (int j = 0; j < S; j++)
						{
							const int iw = pad_w + j + ow * stride_w;
							if (iw < 0 || iw >= W)
								continue;
							const float *xp = x + (((size_t) n * H + ih) * W + iw) * C;
							const float *wp = wt + ((size_t) i * S + j) * C * K + k0;
							for (int c = 0; c < C; c++)
							{
								const float xv = xp[c];
								const float *wr = wp + (size_t) c * K;
#pragma omp simd
								for (int k = 0; k < kn; k++)
									acc[k] += xv * wr[k];
							}
						}
					}
					for (int k = 0; k < kn; k++)
						yp[k0 + k] = (relu && acc[k] < 0.0f) ? 0.0f : acc[k];
				}
			}
		}
	free(wt);
	return 0;
}

/* int8 counterpart of the timed baseline: int32 accumulation, y = acc + bias. */
int orc_conv2d_i8_omp(const int8_t *x, const int8_t *w, const int32_t *bias, int32_t *y, int N, int H, int W, int C, int K, int R, int S, int Ho,
		int Wo, int pad_h, int pad_w, int stride_h, int stride_w)
{
	int16_t *wt = (int16_t*) malloc(sizeof(int16_t) * (size_t) R * S * C * K);
	if (wt == NULL)
		return -1;
	for (int k = 0; k < K; k++)
		for (int i = 0; i < R; i++)
			for (int j = 0; j < S; j++)
				for (int c = 0; c < C; c++)
					wt[(((size_t) i * S + j) * C + c) * K + k] = w[(((size_t) k * R + i) * S + j) * C + c];
#pragma omp parallel for collapse(2) schedule(static)
	for (int n = 0; n < N; n++)
		for (int oh = 0; oh < Ho; oh++)
		{
			int32_t acc[1024];
			for (int ow = 0; ow < Wo; ow++)
			{
				int32_t *yp = y + (((size_t) n * Ho + oh) * Wo + ow) * K;
				for (int k0 = 0; k0 < K; k0 += 1024)
				{
					const int kn = (K - k0) < 1024 ? (K - k0) : 1024;
					for (int k = 0; k < kn; k++)
						acc[k] = bias != NULL ? bias[k0 + k] : 0;
					for (int i = 0; i < R; i++)
					{
						const int ih = pad_h + i + oh * stride_h;
						if (ih < 0 || ih >= H)
							continue;
						for (int j = 0; j < S; j++)
						{
							const int iw = pad_w + j + ow * stride_w;
							if (iw < 0 || iw >= W)
								continue;
							const int8_t *xp = x + (((size_t) n * H + ih) * W + iw) * C;
							const int16_t *wp = wt + ((size_t) i * S + j) * C * K + k0;
							for (int c = 0; c < C; c++)
							{
								const int32_t xv = xp[c];
								const int16_t *wr = wp + (size_t) c * K;
#pragma omp simd
								for (int k = 0; k < kn; k++)
									acc[k] += xv * (int32_t) wr[k];
							}
						}
					}
					for (int k = 0; k < kn; k++)
						yp[k0 + k] = acc[k];
				}
			}
		}
	free(wt);
	return 0;
}

int orc_num_threads(void)
{
#ifdef _OPENMP
	extern int omp_get_max_threads(void);
	return omp_get_max_threads();
#else
	return 1;
#endif
}
