/*
 * avocado_oracle.c  --  TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the convolution hot path of AvocadoML/CudaBackend, used as the parity
 * checker by tests/, by the smoke check and by the cpu_baseline leg of bench.py.  Nothing the
 * product ships may call, link or import this file: the product path is the HIP library and it
 * fails loudly when that library is missing.
 *
 * Every floating-point routine works on double arrays with double accumulation (callers round
 * their inputs to the tensor dtype first and widen them), every integer routine is exact.
 * The timed CPU baseline lives in cpu_baseline.c and is not a checker.
 *
 * What pins each function (the reference ships no golden vectors and its own CPU backend is a
 * separate project that is not available):
 *   orc_conv2d_f64            pinned: torch.nn.functional.conv2d in fp64, hand-computed tiny cases,
 *                             delta-kernel / all-ones / linearity / 1x1==matmul invariants.
 *   orc_conv2d_i8             pinned: exact integer arithmetic against numpy int64 einsum and the
 *                             fp64 routine (exact for these magnitudes).
 *   orc_requant_i8            pinned: hand-written table of exact products (ties to even, saturation at both
 *                             ends, the int32 -> fp32 rounding of the sum, per-filter scale).  The reference has no
 *                             requantisation step; the definition is the benchmark's:
 *                             q = sat_i8(rne(float(sum + bias) * scale[k])), each step one fp32 rounding.
 *   orc_winograd_*_transform  pinned: A^T[(G g G^T) .* (B^T d B)]A == direct correlation to 1e-12
 *                             for every (m, r) table, partial tiles and offsets included.
 *   orc_winograd_gradient_transform, orc_winograd_update_transform
 *                             pinned: U'[(G' dy G'^T) .* (B^T d B)]U'^T == the r x r correlation of the input tile d
 *                             with the m x m tile dy to 1e-12 for every (m, r); a whole weight gradient assembled from
 *                             them equals torch's fp64 autograd weight gradient of conv2d.
 *   orc_gemm_batched          pinned: numpy matmul / einsum on all four (N|T, N|T) combinations.
 *                             (The reference delegates to cuBLAS, whose source is not part of it.)
 *   orc_add_bias              pinned: numpy restatement of the documented formula in two algebraic
 *                             forms; operation order from the reference kernel.
 *   orc_im2row                pinned: rows times flattened weights == orc_conv2d_f64, strides and dilations included
 *                             (the reference's kernel is stride 1 only; its strided test cases are commented out,
 *                             test/test_im2row.cpp:31-48).
 *   orc_affine_forward        pinned: with weight 1 it is orc_add_bias (itself pinned); numpy broadcast form.
 *   orc_batchnorm_inference   pinned: torch.nn.functional.batch_norm(training=False) in fp64; equals
 *                             orc_affine_forward on the folded parameters.
 *   orc_conv2d_i8_float_epilogue  pinned: with alpha1 = 1 and integer-valued terms below 2^24 it equals the exact
 *                             integer routine bit for bit (int32, int8 after clamping, fp32); hand-written cases for
 *                             ties, saturation of int8 and int32, NaN, infinities, the separate fp32 roundings of
 *                             product / bias / residual (a fused multiply-add or a wider intermediate fails them)
 *                             and the order of the steps (every other order fails a case).
 *                             Deviation, stated: the reference kernel stores the float through C's implicit
 *                             conversion (toward zero, src/conv2d_implicit_gemm.cu:285); this build rounds to nearest
 *                             even and saturates, as its cudaChangeType and the requantised output do.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   app/CudaBackend.cu:122-201               direct convolution loop nest, offset padding
 *   include/Avocado/cuda_backend.h:796,822,877  y = act(alpha1*conv + alpha2*z + b) + beta*y
 *   src/winograd_nonfused.cu:220-254         M * tile * M^T algebra of first/second transform
 *   src/winograd_nonfused.cu:303-423         tiling, padding, clipping, epilogue order
 *   src/winograd_nonfused.cu:425-519         gradient and update transforms of the weight gradient
 *   src/winograd_nonfused.cu:534-575         transform coefficient tables
 *   src/activations.cuh:30-121               NHWC offsets, tile index, [t*t, tiles, C] matrices
 *   src/activations.cuh:202-456              activation functions
 *   src/tensor_op.cu:199-228                 add-bias operation order
 *   src/gemm.cpp:126-145                     batched GEMM operand/shape mapping
 *   src/im2row.cu:29-66                      im2row slot order
 *   src/batchnorm.cu:28-69                   affine forward and batch normalisation in inference
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum
{
	ACT_LINEAR = 0, ACT_SIGMOID, ACT_TANH, ACT_RELU, ACT_SELU, ACT_ELU, ACT_EXPONENTIAL, ACT_SOFTPLUS, ACT_SOFTSIGN
};

/* src/activations.cuh:202-425 (forward functions only). */
static double activation_forward(int act, double x)
{
	switch (act)
	{
		default:
		case ACT_LINEAR:
			return x;
		case ACT_SIGMOID:
			return 1.0 / (1.0 + exp(-x));
		case ACT_TANH:
			return tanh(x);
		case ACT_RELU:
			return x > 0.0 ? x : 0.0;
		case ACT_SELU:
			return 1.05070098 * (x >= 0.0 ? x : 1.67326324 * expm1(x));
		case ACT_ELU:
			return x >= 0.0 ? x : expm1(x);
		case ACT_EXPONENTIAL:
			return exp(x);
		case ACT_SOFTPLUS:
			return log1p(exp(x));
		case ACT_SOFTSIGN:
			return x / (fabs(x) + 1.0);
	}
}

double orc_activation(int act, double x)
{
	return activation_forward(act, x);
}

/*
 * Direct convolution, NHWC, weights [K, R, S, C/groups], app/CudaBackend.cu:122-201.
 * pad_* are signed input offsets ("3x3 pad 1" is -1, test/test_im2row.cpp:20).
 * mode 0 = AVOCADO_CONVOLUTION_MODE (kernel used as stored), 1 = AVOCADO_CROSS_CORRELATION_MODE
 * (kernel flipped by 180 degrees, app/CudaBackend.cu:175-179, src/winograd_nonfused.cu:616).
 * Epilogue in the order of src/winograd_nonfused.cu:407-417:
 *   t = alpha1*conv; t += bias[k]; t += alpha2*z; t = act(t); t += beta*y_old.
 * bias and z may be NULL; y is read only when beta != 0.
 */
void orc_conv2d_f64(const double *x, const double *w, const double *bias, const double *z, double *y, int N, int H, int W, int C, int K, int R,
		int S, int Ho, int Wo, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int groups, int mode, double padding_value,
		double alpha1, double alpha2, double beta, int activation)
{
	const int Cg = C / groups; /* input channels per group == last dim of w */
	const int Kg = K / groups;
#pragma omp parallel for collapse(2) schedule(static)
	for (int n = 0; n < N; n++)
		for (int oh = 0; oh < Ho; oh++)
			for (int ow = 0; ow < Wo; ow++)
				for (int k = 0; k < K; k++)
				{
					const int g = k / Kg;
					double acc = 0.0;
					for (int i = 0; i < R; i++)
						for (int j = 0; j < S; j++)
						{
							const int ii = (mode == 0) ? i : (R - 1 - i);
							const int jj = (mode == 0) ? j : (S - 1 - j);
							const int ih = pad_h + ii * dil_h + oh * stride_h;
							const int iw = pad_w + jj * dil_w + ow * stride_w;
							const double *wp = w + (((size_t) k * R + i) * S + j) * Cg;
							if (ih >= 0 && ih < H && iw >= 0 && iw < W)
							{
								const double *xp = x + (((size_t) n * H + ih) * W + iw) * C + (size_t) g * Cg;
								for (int c = 0; c < Cg; c++)
									acc += wp[c] * xp[c];
							}
							else
							{
								for (int c = 0; c < Cg; c++)
									acc += wp[c] * padding_value;
							}
						}
					const size_t idx = (((size_t) n * Ho + oh) * Wo + ow) * K + k;
					double t = alpha1 * acc;
					if (bias != NULL)
						t += bias[k];
					if (z != NULL)
						t += alpha2 * z[idx];
					t = activation_forward(activation, t);
					if (beta != 0.0)
						t += beta * y[idx];
					y[idx] = t;
				}
}

/*
 * Quantised direct convolution: int8 activations and weights, exact integer accumulation,
 * y = act(acc + bias[k]) as int32 (activation is LINEAR or RELU), groups = 1.
 * Same loop nest and offset padding as orc_conv2d_f64; padding value is an int8.
 */
void orc_conv2d_i8(const int8_t *x, const int8_t *w, const int32_t *bias, int32_t *y, int N, int H, int W, int C, int K, int R, int S, int Ho,
		int Wo, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int mode, int padding_value, int activation)
{
#pragma omp parallel for collapse(2) schedule(static)
	for (int n = 0; n < N; n++)
		for (int oh = 0; oh < Ho; oh++)
			for (int ow = 0; ow < Wo; ow++)
				for (int k = 0; k < K; k++)
				{
					int64_t acc = 0;
					for (int i = 0; i < R; i++)
						for (int j = 0; j < S; j++)
						{
							const int ii = (mode == 0) ? i : (R - 1 - i);
							const int jj = (mode == 0) ? j : (S - 1 - j);
							const int ih = pad_h + ii * dil_h + oh * stride_h;
							const int iw = pad_w + jj * dil_w + ow * stride_w;
							const int8_t *wp = w + (((size_t) k * R + i) * S + j) * C;
							if (ih >= 0 && ih < H && iw >= 0 && iw < W)
							{
								const int8_t *xp = x + (((size_t) n * H + ih) * W + iw) * C;
								for (int c = 0; c < C; c++)
									acc += (int64_t) wp[c] * (int64_t) xp[c];
							}
							else
							{
								for (int c = 0; c < C; c++)
									acc += (int64_t) wp[c] * (int64_t) padding_value;
							}
						}
					if (bias != NULL)
						acc += bias[k];
					if (activation == ACT_RELU && acc < 0)
						acc = 0;
					y[(((size_t) n * Ho + oh) * Wo + ow) * K + k] = (int32_t) acc;
				}
}

static inline int32_t saturate_round(float v, int32_t lo, int32_t hi)
{
	if (!(v == v)) /* NaN */
		return 0;
	float r = nearbyintf(v); /* default rounding mode: nearest even */
	if (r < (float) lo)
		return lo;
	if (r >= (float) hi) /* (float) INT32_MAX is 2^31: everything from there up saturates */
		return hi;
	return (int32_t) r;
}

/*
 * Requantisation of an int32 accumulator tensor [rows, K] (bias already added) to int8:
 * q = saturate_i8(round_nearest_even(float(acc) * scale[k])), every step one IEEE-754 fp32 rounding.
 * Build with -ffp-contract=off.
 */
void orc_requant_i8(const int32_t *acc, const float *scale, int8_t *q, int64_t rows, int K)
{
	for (int64_t r = 0; r < rows; r++)
		for (int k = 0; k < K; k++)
		{
			const float v = (float) acc[r * K + k] * scale[k];
			q[r * K + k] = (int8_t) saturate_round(v, -128, 127);
		}
}

/*
 * Float epilogue on an integer accumulator (include/Avocado/cuda_backend.h:43-49: integer tensors
 * are cast to fp32, scaled in fp32 and cast back).  acc is the raw int32 convolution sum without bias.
 *   t = alpha1*float(acc); t += bias[k]; t += alpha2*float(z); t = act(t); t += beta*float(y_old)
 * out_kind: 0 -> int32 (round to nearest even, saturate), 1 -> int8 (same), 2 -> fp32.
 */
void orc_conv2d_i8_float_epilogue(const int32_t *acc, const float *bias, const void *z, void *y, int64_t rows, int K, float alpha1, float alpha2,
		float beta, int activation, int out_kind)
{
	for (int64_t r = 0; r < rows; r++)
		for (int k = 0; k < K; k++)
		{
			const int64_t idx = r * K + k;
			float t = alpha1 * (float) acc[idx];
			if (bias != NULL)
				t = t + bias[k];
			if (z != NULL)
			{
				float zv = (out_kind == 0) ? (float) ((const int32_t*) z)[idx] : (out_kind == 1) ? (float) ((const int8_t*) z)[idx] : ((const float*) z)[idx];
				t = t + alpha2 * zv;
			}
			t = (float) activation_forward(activation, (double) t);
			if (beta != 0.0f)
			{
				float yv = (out_kind == 0) ? (float) ((int32_t*) y)[idx] : (out_kind == 1) ? (float) ((int8_t*) y)[idx] : ((float*) y)[idx];
				t = t + beta * yv;
			}
			if (out_kind == 0)
				((int32_t*) y)[idx] = saturate_round(t, INT32_MIN, INT32_MAX);
			else if (out_kind == 1)
				((int8_t*) y)[idx] = (int8_t) saturate_round(t, -128, 127);
			else
				((float*) y)[idx] = t;
		}
}

/* ---------------------------------------------------------------------------------------------
 * Winograd transform tables, src/winograd_nonfused.cu:534-575.  Row-major.
 *   weight  G   : t x r      input  B^T : t x t      output  A^T : m x t      (t = m + r - 1)
 * --------------------------------------------------------------------------------------------- */
#define T3 (1.0 / 3.0)
static const double G_2_3[4 * 3] = { 1, 0, 0, 1, 1, 1, 1, -1, 1, 0, 0, 1 };
static const double BT_2_3[4 * 4] = { 1, 0, -1, 0, 0, 1, 1, 0, 0, -1, 1, 0, 0, -1, 0, 1 };
static const double AT_2_3[2 * 4] = { 1, 0.5, 0.5, 0, 0, 0.5, -0.5, 1 };

static const double G_4_3[6 * 3] = { 1, 0, 0, 2 * T3, 2 * T3, 2 * T3, 2 * T3, -2 * T3, 2 * T3, T3, 2 * T3, 4 * T3, T3, -2 * T3, 4 * T3, 0, 0, 2 };
static const double BT_6[6 * 6] = { 1, 0, -1.25, 0, 0.25, 0, 0, 1, 1, -0.25, -0.25, 0, 0, -1, 1, 0.25, -0.25, 0, 0, -1, -0.5, 1, 0.5, 0, 0, 1, -0.5, -1,
		0.5, 0, 0, 1, 0, -1.25, 0, 0.25 };
static const double AT_4_3[4 * 6] = { 1, 1, 1, 0.25, 0.25, 0, 0, 1, -1, 0.5, -0.5, 0, 0, 1, 1, 1, 1, 0, 0, 1, -1, 2, -2, 2 };

static const double G_2_5[6 * 5] = { 1, 0, 0, 0, 0, 2 * T3, 2 * T3, 2 * T3, 2 * T3, 2 * T3, 2 * T3, -2 * T3, 2 * T3, -2 * T3, 2 * T3, T3 / 2, T3, 2 * T3,
		4 * T3, 8 * T3, T3 / 2, -T3, 2 * T3, -4 * T3, 8 * T3, 0, 0, 0, 0, 2 };
static const double AT_2_5[2 * 6] = { 1, 1, 1, 0.5, 0.5, 0, 0, 1, -1, 1, -1, 2 };

/* Weight-gradient side (src/winograd_nonfused.cu:538-539,558-562,571-574): gradient G' [t x m], update U' [r x t]. */
static const double GR_2_3[4 * 2] = { 1, 0, 1, 1, 1, -1, 0, 1 };
static const double UP_2_3[3 * 4] = { 1, 0.5, 0.5, 0, 0, 0.5, -0.5, 0, 0, 0.5, 0.5, 1 };
static const double GR_4_3[6 * 4] = { 1, 0, 0, 0, 2 * T3, 2 * T3, 2 * T3, 2 * T3, 2 * T3, -2 * T3, 2 * T3, -2 * T3, T3, 2 * T3, 4 * T3, 8 * T3, T3, -2 * T3,
	4 * T3, -8 * T3, 0, 0, 0, 2 };
static const double UP_4_3[3 * 6] = { 1, 1, 1, 0.25, 0.25, 0, 0, 1, -1, 0.5, -0.5, 0, 0, 1, 1, 1, 1, 2 };
static const double GR_2_5[6 * 2] = { 1, 0, 2 * T3, 2 * T3, 2 * T3, -2 * T3, T3, 2 * T3, T3, -2 * T3, 0, 1 };
static const double UP_2_5[5 * 6] = { 1, 1, 1, 0.25, 0.25, 0, 0, 1, -1, 0.5, -0.5, 0, 0, 1, 1, 1, 1, 0, 0, 1, -1, 2, -2, 0, 0, 1, 1, 4, 4, 4 };

static int get_training_tables(int m, int r, const double **GR, const double **UP)
{
	if (m == 2 && r == 3)
	{
		*GR = GR_2_3;
		*UP = UP_2_3;
		return 0;
	}
	if (m == 4 && r == 3)
	{
		*GR = GR_4_3;
		*UP = UP_4_3;
		return 0;
	}
	if (m == 2 && r == 5)
	{
		*GR = GR_2_5;
		*UP = UP_2_5;
		return 0;
	}
	return -1;
}

/* Returns 0 when (m, r) is one of the three supported pairs, src/winograd_nonfused.cu:626-650. */
static int get_tables(int m, int r, const double **G, const double **BT, const double **AT)
{
	if (m == 2 && r == 3)
	{
		*G = G_2_3;
		*BT = BT_2_3;
		*AT = AT_2_3;
		return 0;
	}
	if (m == 4 && r == 3)
	{
		*G = G_4_3;
		*BT = BT_6;
		*AT = AT_4_3;
		return 0;
	}
	if (m == 2 && r == 5)
	{
		*G = G_2_5;
		*BT = BT_6;
		*AT = AT_2_5;
		return 0;
	}
	return -1;
}

/* Copies a table out (which: 0 = G, 1 = B^T, 2 = A^T, 3 = gradient, 4 = update); returns the number of coefficients or -1. */
int orc_winograd_table(int m, int r, int which, double *out)
{
	const double *G, *BT, *AT, *GR, *UP;
	if (get_tables(m, r, &G, &BT, &AT) != 0 || get_training_tables(m, r, &GR, &UP) != 0 || which < 0 || which > 4)
		return -1;
	const int t = m + r - 1;
	const double *src = which == 0 ? G : which == 1 ? BT : which == 2 ? AT : which == 3 ? GR : UP;
	const int n = which == 0 ? t * r : which == 1 ? t * t : which == 2 ? m * t : which == 3 ? t * m : r * t;
	memcpy(out, src, sizeof(double) * n);
	return n;
}

/* out[rows_m x rows_m] = Mx[rows_m x cols_m] * tile[cols_m x cols_m] * Mx^T, src/winograd_nonfused.cu:220-254. */
static void sandwich(const double *Mx, int rows_m, int cols_m, const double *tile, double *out)
{
	double tmp[8 * 8];
	for (int i = 0; i < rows_m; i++)
		for (int j = 0; j < cols_m; j++)
		{
			double s = 0.0;
			for (int k = 0; k < cols_m; k++)
				s += Mx[i * cols_m + k] * tile[k * cols_m + j];
			tmp[i * cols_m + j] = s;
		}
	for (int i = 0; i < rows_m; i++)
		for (int j = 0; j < rows_m; j++)
		{
			double s = 0.0;
			for (int k = 0; k < cols_m; k++)
				s += tmp[i * cols_m + k] * Mx[j * cols_m + k];
			out[i * rows_m + j] = s;
		}
}

/*
 * U[(i*t+j), k, c] = (G g[k,:,:,c] G^T)[i,j]; invert != 0 flips g by 180 degrees first
 * (src/winograd_nonfused.cu:257-301, :616).  w is [K, r, r, C], U is [t*t, K, C].
 */
int orc_winograd_weight_transform(const double *w, double *U, int K, int C, int m, int r, int invert)
{
	const double *G, *BT, *AT;
	if (get_tables(m, r, &G, &BT, &AT) != 0)
		return -1;
	const int t = m + r - 1;
	for (int k = 0; k < K; k++)
		for (int c = 0; c < C; c++)
		{
			double g[5 * 5], out[8 * 8];
			for (int i = 0; i < r; i++)
				for (int j = 0; j < r; j++)
				{
					const double v = w[(((size_t) k * r + i) * r + j) * C + c];
					if (invert)
						g[(r - 1 - i) * r + (r - 1 - j)] = v;
					else
						g[i * r + j] = v;
				}
			sandwich(G, t, r, g, out);
			for (int i = 0; i < t * t; i++)
				U[((size_t) i * K + k) * C + c] = out[i];
		}
	return 0;
}

/*
 * V[(i*t+j), tile, c] = (B^T d B)[i,j], d[a,b] = x[n, pad_h + th*m + a, pad_w + tw*m + b, c] or
 * padding_value outside the image; tile = (n*Th + th)*Tw + tw, Th = ceil(H/m), Tw = ceil(W/m)
 * (src/winograd_nonfused.cu:303-365, src/activations.cuh:52-68).
 */
int orc_winograd_input_transform(const double *x, double *V, int N, int H, int W, int C, int m, int r, int pad_h, int pad_w, double padding_value)
{
	const double *G, *BT, *AT;
	if (get_tables(m, r, &G, &BT, &AT) != 0)
		return -1;
	const int t = m + r - 1;
	const int Th = (H + m - 1) / m, Tw = (W + m - 1) / m;
	const size_t tiles = (size_t) N * Th * Tw;
#pragma omp parallel for collapse(2) schedule(static)
	for (int n = 0; n < N; n++)
		for (int th = 0; th < Th; th++)
			for (int tw = 0; tw < Tw; tw++)
				for (int c = 0; c < C; c++)
				{
					double d[8 * 8], out[8 * 8];
					for (int a = 0; a < t; a++)
						for (int b = 0; b < t; b++)
						{
							const int ih = pad_h + th * m + a;
							const int iw = pad_w + tw * m + b;
							d[a * t + b] = (ih >= 0 && ih < H && iw >= 0 && iw < W) ? x[(((size_t) n * H + ih) * W + iw) * C + c] : padding_value;
						}
					sandwich(BT, t, t, d, out);
					const size_t tile = ((size_t) n * Th + th) * Tw + tw;
					for (int i = 0; i < t * t; i++)
						V[((size_t) i * tiles + tile) * C + c] = out[i];
				}
	return 0;
}

/*
 * y[n, th*m + a, tw*m + b, k] = act(alpha1*(A^T M A)[a,b] + bias[k] + alpha2*z) + beta*y_old, clipped
 * to H x W (src/winograd_nonfused.cu:366-423).  Mx is [t*t, tiles, K]; y, z are [N, H, W, K].
 */
int orc_winograd_output_transform(const double *Mx, double *y, const double *bias, const double *z, int N, int H, int W, int K, int m, int r,
		double alpha1, double alpha2, double beta, int activation)
{
	const double *G, *BT, *AT;
	if (get_tables(m, r, &G, &BT, &AT) != 0)
		return -1;
	const int t = m + r - 1;
	const int Th = (H + m - 1) / m, Tw = (W + m - 1) / m;
	const size_t tiles = (size_t) N * Th * Tw;
#pragma omp parallel for collapse(2) schedule(static)
	for (int n = 0; n < N; n++)
		for (int th = 0; th < Th; th++)
			for (int tw = 0; tw < Tw; tw++)
				for (int k = 0; k < K; k++)
				{
					double d[8 * 8], tmp[8 * 8];
					const size_t tile = ((size_t) n * Th + th) * Tw + tw;
					for (int i = 0; i < t * t; i++)
						d[i] = Mx[((size_t) i * tiles + tile) * K + k];
					/* tmp[m x t] = A^T d ; out[a,b] = sum_j tmp[a,j] * A^T[b,j] */
					for (int a = 0; a < m; a++)
						for (int j = 0; j < t; j++)
						{
							double s = 0.0;
							for (int q = 0; q < t; q++)
								s += AT[a * t + q] * d[q * t + j];
							tmp[a * t + j] = s;
						}
					for (int a = 0; a < m; a++)
						for (int b = 0; b < m; b++)
						{
							const int oh = th * m + a, ow = tw * m + b;
							if (oh >= H || ow >= W)
								continue;
							double s = 0.0;
							for (int j = 0; j < t; j++)
								s += tmp[a * t + j] * AT[b * t + j];
							const size_t idx = (((size_t) n * H + oh) * W + ow) * K + k;
							double v = alpha1 * s;
							if (bias != NULL)
								v += bias[k];
							if (z != NULL)
								v += alpha2 * z[idx];
							v = activation_forward(activation, v);
							if (beta != 0.0)
								v += beta * y[idx];
							y[idx] = v;
						}
				}
	return 0;
}

/*
 * Mx[(i*t+j), tile, k] = (G' d G'^T)[i,j], d[a,b] = dy[n, th*m + a, tw*m + b, k] or 0 past the border; tiles do not overlap,
 * tile = (n*Th + th)*Tw + tw (src/winograd_nonfused.cu:425-474).  dy is [N, H, W, K], Mx is [t*t, tiles, K].
 */
int orc_winograd_gradient_transform(const double *dy, double *Mx, int N, int H, int W, int K, int m, int r)
{
	const double *GR, *UP;
	if (get_training_tables(m, r, &GR, &UP) != 0)
		return -1;
	const int t = m + r - 1;
	const int Th = (H + m - 1) / m, Tw = (W + m - 1) / m;
	const size_t tiles = (size_t) N * Th * Tw;
	for (int n = 0; n < N; n++)
		for (int th = 0; th < Th; th++)
			for (int tw = 0; tw < Tw; tw++)
				for (int k = 0; k < K; k++)
				{
					double d[8 * 8], out[8 * 8];
					for (int a = 0; a < m; a++)
						for (int b = 0; b < m; b++)
						{
							const int h = th * m + a, w = tw * m + b;
							d[a * m + b] = (h < H && w < W) ? dy[(((size_t) n * H + h) * W + w) * K + k] : 0.0;
						}
					sandwich(GR, t, m, d, out);
					const size_t tile = ((size_t) n * Th + th) * Tw + tw;
					for (int i = 0; i < t * t; i++)
						Mx[((size_t) i * tiles + tile) * K + k] = out[i];
				}
	return 0;
}

/*
 * dw[k, i, j, c] = alpha * (U' d U'^T)[i,j] + beta * dw_old, d = the t x t tile Mx[:, k, c]
 * (src/winograd_nonfused.cu:475-519).  Mx is [t*t, K, C], dw is [K, r, r, C].
 */
int orc_winograd_update_transform(const double *Mx, double *dw, int K, int C, int m, int r, double alpha, double beta)
{
	const double *GR, *UP;
	if (get_training_tables(m, r, &GR, &UP) != 0)
		return -1;
	const int t = m + r - 1;
	for (int k = 0; k < K; k++)
		for (int c = 0; c < C; c++)
		{
			double d[8 * 8], out[8 * 8];
			for (int i = 0; i < t * t; i++)
				d[i] = Mx[((size_t) i * K + k) * C + c];
			sandwich(UP, r, t, d, out);
			for (int i = 0; i < r * r; i++)
			{
				const size_t idx = ((size_t) k * r * r + i) * C + c;
				double v = alpha * out[i];
				if (beta != 0.0)
					v += beta * dw[idx];
				dw[idx] = v;
			}
		}
	return 0;
}

/*
 * C[b] = alpha * op(A[b]) op(B[b]) + beta * C[b], row-major, all batches the same shape
 * (src/gemm.cpp:126-145: batch = first dim, per-batch stride = volume without the first dim).
 * A[b] is (opA ? KxM : MxK), B[b] is (opB ? NxK : KxN), C[b] is MxN.
 */
void orc_gemm_batched(const double *A, const double *B, double *C, int batch, int M, int N, int K, int opA, int opB, double alpha, double beta)
{
#pragma omp parallel for collapse(2) schedule(static)
	for (int b = 0; b < batch; b++)
		for (int i = 0; i < M; i++)
		{
			const double *a = A + (size_t) b * M * K;
			const double *bb = B + (size_t) b * N * K;
			double *c = C + (size_t) b * M * N;
			for (int j = 0; j < N; j++)
			{
				double s = 0.0;
				for (int k = 0; k < K; k++)
				{
					const double av = opA ? a[(size_t) k * M + i] : a[(size_t) i * K + k];
					const double bv = opB ? bb[(size_t) j * K + k] : bb[(size_t) k * N + j];
					s += av * bv;
				}
				double v = alpha * s;
				if (beta != 0.0)
					v += beta * c[(size_t) i * N + j];
				c[(size_t) i * N + j] = v;
			}
		}
}

/*
 * y = alpha1 * act(alpha2*x + b + beta1*z) + beta2*z + beta3*y, b broadcast over the last dimension
 * (include/Avocado/cuda_backend.h:353, order of operations src/tensor_op.cu:213-226).
 * z is read only when beta1 != 0 or beta2 != 0; y only when beta3 != 0.
 */
void orc_add_bias(const double *x, const double *b, const double *z, double *y, int64_t first, int last, double alpha1, double alpha2, double beta1,
		double beta2, double beta3, int activation)
{
	for (int64_t i = 0; i < first; i++)
		for (int j = 0; j < last; j++)
		{
			const int64_t idx = i * last + j;
			double t = alpha2 * x[idx] + b[j];
			if (beta1 != 0.0 || beta2 != 0.0)
				t = alpha1 * activation_forward(activation, t + beta1 * z[idx]) + beta2 * z[idx];
			else
				t = alpha1 * activation_forward(activation, t);
			if (beta3 != 0.0)
				t += beta3 * y[idx];
			y[idx] = t;
		}
}

/*
 * y = alpha * act(x * weight[j] + bias[j]) + beta * y over a [first, last] view (src/batchnorm.cu:28-48).
 */
void orc_affine_forward(const double *x, const double *weight, const double *bias, double *y, int64_t first, int64_t last, double alpha, double beta,
		int activation)
{
	for (int64_t i = 0; i < first; i++)
		for (int64_t j = 0; j < last; j++)
		{
			const int64_t idx = i * last + j;
			double t = alpha * activation_forward(activation, x[idx] * weight[j] + bias[j]);
			if (beta != 0.0)
				t += beta * y[idx];
			y[idx] = t;
		}
}

/*
 * Batch normalisation with stored statistics (src/batchnorm.cu:51-69): per channel j
 *   s = scale[j] / sqrt(variance[j] + epsilon),  t = bias[j] - mean[j] * s,  y = alpha * act(x * s + t) + beta * y.
 */
void orc_batchnorm_inference(const double *x, const double *scale, const double *bias, const double *mean, const double *variance, double *y,
		int64_t first, int64_t last, double alpha, double beta, double epsilon, int activation)
{
	for (int64_t j = 0; j < last; j++)
	{
		const double s = scale[j] / sqrt(variance[j] + epsilon);
		const double t = bias[j] - mean[j] * s;
		for (int64_t i = 0; i < first; i++)
		{
			const int64_t idx = i * last + j;
			double r = alpha * activation_forward(activation, x[idx] * s + t);
			if (beta != 0.0)
				r += beta * y[idx];
			y[idx] = r;
		}
	}
}

/*
 * Explicit im2row: rows[(n*Ho + oh)*Wo + ow, (i*S + j)*C + c] = x[n, pad_h + oh + i', pad_w + ow + j', c]
 * or padding_value outside, stride 1, dilation 1; (i', j') = (i, j) in convolution mode and the
 * flipped tap in cross-correlation mode, so that rows x flattened-weights^T reproduces the convolution
 * (slot order of src/im2row.cu:47-62 expressed per output pixel).
 */
void orc_im2row(const double *x, double *rows, int N, int H, int W, int C, int R, int S, int Ho, int Wo, int pad_h, int pad_w, int stride_h,
		int stride_w, int dil_h, int dil_w, int mode, double padding_value)
{
	for (int n = 0; n < N; n++)
		for (int oh = 0; oh < Ho; oh++)
			for (int ow = 0; ow < Wo; ow++)
				for (int i = 0; i < R; i++)
					for (int j = 0; j < S; j++)
					{
						const int ii = (mode == 0) ? i : (R - 1 - i);
						const int jj = (mode == 0) ? j : (S - 1 - j);
						const int ih = pad_h + oh * stride_h + ii * dil_h, iw = pad_w + ow * stride_w + jj * dil_w;
						double *dst = rows + ((((size_t) n * Ho + oh) * Wo + ow) * R * S + (size_t) i * S + j) * C;
						for (int c = 0; c < C; c++)
							dst[c] = (ih >= 0 && ih < H && iw >= 0 && iw < W) ? x[(((size_t) n * H + ih) * W + iw) * C + c] : padding_value;
					}
}
