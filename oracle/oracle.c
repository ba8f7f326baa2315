/* oracle.c — CPU restatement of the reference CPU math engine for the inference hot path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the shipped library links, loads or calls this file; it is the checker
 * that tests, the smoke run and the benchmark's cpu_baseline leg compare the HIP kernels against.
 *
 * Plain scalar C, fp32 arithmetic (long dot products - matrix products, convolution, LSTM gate sums - accumulate in
 * double and round once: the reference's fp32 result depends on its blocking order, and both it and the GPU result are
 * compared with the correctly rounded value), loops written from the definitions the reference uses
 * (paths below are relative to /root/reference/NeoMathEngine/):
 *   - convolution            test/src/common/MeTestCommon.h:67-105 (batchConvolutionForward),
 *                            output size src/CPU/CpuMathEngineDnnConv.cpp:59-62
 *   - channelwise conv       test/src/inference/BlobChannelwiseConvolutionTest.cpp:21-70
 *   - matrix products        test/src/inference/MultiplyMatrixByTransposedMatrixTest.cpp:21-37,
 *                            test/src/common/MeTestCommon.h:34-53,
 *                            test/src/learn/MultiplyTransposedMatrixByMatrixTest.cpp:21-36
 *   - max pooling (+index)   src/CPU/CpuMathEngineDnnPooling.cpp:40-84, src/CPU/CpuMathEngineBlas.cpp:784-806
 *   - mean pooling           src/CPU/CpuMathEngineDnnPooling.h:23-70
 *   - element-wise ops       src/CPU/x86/CpuX86MathEngineVectorMath.cpp:320-337,1321-1366,
 *                            src/CPU/x86/CpuX86MathEngineVectorMathMkl.cpp:46-121,
 *                            src/CPU/x86/CpuX86MathEngineVectorMathPrivate.h:1178-1260, src/CPU/x86/CpuX86.h:55
 *   - broadcasts / sums      src/CPU/CpuMathEngineBlas.cpp:216-252,324-409,808-823,954-
 *   - softmax                src/CPU/CpuMathEngineBlas.cpp:1131-1159
 *   - arg-max                test/src/inference/FindMaxValueInRowsTest.cpp:37-50 (first index on ties),
 *                            src/CPU/x86/CpuX86MathEngineBlas.cpp:183-246 (columns)
 *   - transpose              src/CPU/CpuMathEngineBlas.cpp:103-150
 *   - split / merge          src/CPU/CpuMathEngineDnn.cpp:62-140
 *   - resize image           src/CPU/Rowwise/CpuRowwiseResizeImage.h:22-195
 *   - LSTM                   src/CPU/CpuMathEngineDnnLstm.cpp:114-211, src/CPU/CpuMathEngineDnnLstm.h:49-90
 *   - CTC greedy collapse    ../NeoML/src/Dnn/Layers/CtcLayer.cpp:342-369
 *
 * Pinning: every function here is checked in tests/test_oracle.py against the reference's own CPU engine built
 * from its sources (oracle/_ref, see oracle/Makefile) and against independent numpy / scipy formulations.
 * Known, documented deviation: orc_find_max_value_in_rows takes the FIRST index on exact ties (the rule of the
 * reference's test); the reference's SSE code resolves exact ties by lane, so ties are kept out of parity inputs.
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------------------ */
/* scalar helpers */

static float orc_exp_clamped(float x)
{
	if (x < -87.33654474f) return 0.f;
	if (x > 88.f) return FLT_MAX;
	return expf(x);
}

/* ------------------------------------------------------------------------------------------------------ */
/* element-wise. op codes shared with tests/opcodes in python (see tests/nhtest.py) */

enum {
	ORC_RELU = 0, ORC_ELU, ORC_LEAKY_RELU, ORC_HSWISH, ORC_ABS, ORC_HARD_TANH, ORC_HARD_SIGMOID, ORC_NEG,
	ORC_EXP, ORC_LOG, ORC_ERF, ORC_SQRT, ORC_INV, ORC_MINMAX, ORC_SIGMOID, ORC_TANH,
	ORC_ADD_VALUE, ORC_MULTIPLY, ORC_NEG_MULTIPLY, ORC_COPY, ORC_NEG_LOG,
	ORC_SUB_VALUE, ORC_VALUE_SUB, /* x - p0 and p0 - x: the scalar forms of VectorSub */
	/* element-wise parts of the losses (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:584-782) */
	ORC_HINGE, ORC_SQUARED_HINGE, ORC_HUBER, ORC_HUBER_DERIVATIVE
};

/* result[i] = f(first[i]; p0, p1) */
ORC_API void orc_vector_unary(int op, const float* first, float* result, int n, float p0, float p1)
{
	for (int i = 0; i < n; ++i) {
		const float x = first[i];
		float y = 0.f;
		switch (op) {
		case ORC_RELU: y = x > 0.f ? x : 0.f; if (p0 > 0.f && y > p0) y = p0; break;
		case ORC_ELU: y = x >= 0.f ? x : p0 * (orc_exp_clamped(x) - 1.f); break;
		case ORC_LEAKY_RELU: y = x > 0.f ? x : p0 * x; break;
		case ORC_HSWISH: y = x <= -3.f ? 0.f : (x >= 3.f ? x : x * (x + 3.f) * (1.f / 6.f)); break;
		case ORC_ABS: y = fabsf(x); break;
		case ORC_HARD_TANH: y = x < -1.f ? -1.f : (x > 1.f ? 1.f : x); break;
		case ORC_HARD_SIGMOID: y = x * p0 + p1; y = y < 0.f ? 0.f : (y > 1.f ? 1.f : y); break;
		case ORC_NEG: y = -x; break;
		case ORC_EXP: y = orc_exp_clamped(x); break;
		case ORC_LOG: { float c = x > FLT_MIN ? x : FLT_MIN; c = c < FLT_MAX ? c : FLT_MAX; y = logf(c); } break;
		case ORC_ERF: y = erff(x); break;
		case ORC_SQRT: y = sqrtf(x); break;
		case ORC_INV:
			/* the reference runs with denormals-are-zero: a denormal of either sign compares as +0 */
			if (fabsf(x) < FLT_MIN) y = FLT_MAX;
			else if (x >= 0.f && x <= FLT_MIN) y = FLT_MAX;
			else if (x < 0.f && x >= -FLT_MIN) y = -FLT_MAX;
			else y = 1.f / x;
			break;
		case ORC_MINMAX: y = x > p0 ? x : p0; y = y < p1 ? y : p1; break;
		case ORC_SIGMOID: { const float e = orc_exp_clamped(x); y = e / (e + 1.f); } break;
		case ORC_TANH: y = -1.f + 2.f / (1.f + orc_exp_clamped(-2.f * x)); break;
		case ORC_ADD_VALUE: y = x + p0; break;
		case ORC_MULTIPLY: y = x * p0; break;
		case ORC_NEG_MULTIPLY: y = -x * p0; break;
		case ORC_COPY: y = x; break;
		/* VectorLog with the sign flipped (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:1692-1720) */
		case ORC_HINGE: y = 1.f - x > 0.f ? 1.f - x : 0.f; break;
		case ORC_SQUARED_HINGE: { const float t = 1.f - x > 0.f ? 1.f - x : 0.f; y = x < -1.f ? -4.f * x : t * t; } break;
		case ORC_HUBER: y = x > 1.f ? x - 0.5f : (x < -1.f ? -x - 0.5f : x * x / 2); break;
		case ORC_HUBER_DERIVATIVE: y = x > 1.f ? 1.f : (x < -1.f ? -1.f : x); break;
		case ORC_SUB_VALUE: y = x - p0; break;
		case ORC_VALUE_SUB: y = p0 - x; break;
		case ORC_NEG_LOG: { float c = x > FLT_MIN ? x : FLT_MIN; c = c < FLT_MAX ? c : FLT_MAX; y = -logf(c); } break;
		default: y = NAN; break;
		}
		result[i] = y;
	}
}

enum {
	ORC_ADD = 0, ORC_SUB, ORC_ELTWISE_MULTIPLY, ORC_ELTWISE_NEG_MULTIPLY, ORC_ELTWISE_DIVIDE, ORC_ELTWISE_MAX,
	ORC_ELTWISE_MIN, ORC_MULTIPLY_AND_ADD, ORC_MULTIPLY_AND_SUB, ORC_ELTWISE_MULTIPLY_ADD,
	/* derivatives of the activations times second; the _OP forms take the activation's output as first
	 * (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:339-395, 433-480, 1377-1520) */
	ORC_RELU_DIFF, ORC_HSWISH_DIFF, ORC_SIGMOID_DIFF, ORC_SIGMOID_DIFF_OP, ORC_TANH_DIFF, ORC_TANH_DIFF_OP,
	/* (:232-318 ELU, p0 = alpha; :394-432 leaky ReLU, p0 = alpha; :783-812 hard tanh; :825-920 hard sigmoid, p0 = slope,
	 * p1 = bias; :550-580 abs) */
	ORC_ELU_DIFF, ORC_ELU_DIFF_OP, ORC_LEAKY_RELU_DIFF, ORC_HARD_TANH_DIFF, ORC_HARD_SIGMOID_DIFF, ORC_HARD_SIGMOID_DIFF_OP,
	ORC_ABS_DIFF,
	/* (:614-649 hinge, :924-975 squared hinge; :1598-1640 L1 regulariser, p0 = threshold, p1 = multiplier) */
	ORC_HINGE_DIFF, ORC_SQUARED_HINGE_DIFF, ORC_L1_DIFF_ADD
};

/* result[i] = f(first[i], second[i]; p0, p1); ORC_ELTWISE_MULTIPLY_ADD reads result[i] as the addend */
ORC_API void orc_vector_binary(int op, const float* first, const float* second, float* result, int n, float p0, float p1)
{
	for (int i = 0; i < n; ++i) {
		const float a = first[i], b = second[i];
		float y = 0.f;
		switch (op) {
		case ORC_ADD: y = a + b; break;
		case ORC_SUB: y = a - b; break;
		case ORC_ELTWISE_MULTIPLY: y = a * b; break;
		case ORC_ELTWISE_NEG_MULTIPLY: y = -a * b; break;
		case ORC_ELTWISE_DIVIDE: y = a / b; break;
		case ORC_ELTWISE_MAX: y = a > b ? a : b; break;
		case ORC_ELTWISE_MIN: y = a < b ? a : b; break;
		case ORC_MULTIPLY_AND_ADD: { volatile float m = b * p0; y = a + m; } break;
		case ORC_MULTIPLY_AND_SUB: { volatile float m = b * p0; y = a - m; } break;
		case ORC_ELTWISE_MULTIPLY_ADD: { volatile float m = a * b; y = result[i] + m; } break;
		case ORC_RELU_DIFF: y = (a > 0.f && (p0 <= 0.f || a < p0)) ? b : 0.f; break;
		case ORC_HSWISH_DIFF: y = !(-3.f < a) ? 0.f : (a < 3.f ? b * (a * (1.f / 3.f) + 0.5f) : b); break;
		case ORC_SIGMOID_DIFF: { const float e = orc_exp_clamped(-a); y = b / (2.f + e + 1.f / e); } break;
		case ORC_SIGMOID_DIFF_OP: y = a * (1.f - a) * b; break;
		case ORC_TANH_DIFF: { const float t = -1.f + 2.f / (1.f + orc_exp_clamped(-2.f * a)); y = b * (1.f - t * t); } break;
		case ORC_TANH_DIFF_OP: y = (1.f - a * a) * b; break;
		case ORC_ELU_DIFF: { const float e = orc_exp_clamped(a); y = e >= 1.f ? b : b * e * p0; } break;
		case ORC_ELU_DIFF_OP: y = a >= 0.f ? b : b * (a + p0); break;
		case ORC_LEAKY_RELU_DIFF: y = a > 0.f ? b : (a < 0.f ? b * p0 : 0.f); break;
		case ORC_HARD_TANH_DIFF: y = (-1.f < a && a < 1.f) ? b : 0.f; break;
		case ORC_HARD_SIGMOID_DIFF: y = (-p1 / p0 < a && a < (1.f - p1) / p0) ? b * p0 : 0.f; break;
		case ORC_HARD_SIGMOID_DIFF_OP: y = (0.f < a && a < 1.f) ? b * p0 : 0.f; break;
		case ORC_ABS_DIFF: y = a > 0.f ? b : -b; break;
		case ORC_HINGE_DIFF: y = a < 1.f ? -b : 0.f; break;
		case ORC_SQUARED_HINGE_DIFF: { const float t = 1.f - a > 0.f ? 1.f - a : 0.f; y = a < -1.f ? -4.f * b : -2.f * t * b; } break;
		case ORC_L1_DIFF_ADD: { const float x = b < -p0 ? -p0 : (b > p0 ? p0 : b); y = a + p1 * x; } break;
		default: y = NAN; break;
		}
		result[i] = y;
	}
}

enum { ORC_INT_ADD = 0, ORC_INT_SUB, ORC_INT_MULTIPLY };
ORC_API void orc_vector_binary_int(int op, const int* first, const int* second, int* result, int n)
{
	for (int i = 0; i < n; ++i) {
		switch (op) {
		case ORC_INT_ADD: result[i] = first[i] + second[i]; break;
		case ORC_INT_SUB: result[i] = first[i] - second[i]; break;
		default: result[i] = first[i] * second[i]; break;
		}
	}
}

ORC_API void orc_vector_convert_float_to_int(const float* from, int* to, int n)
{
	for (int i = 0; i < n; ++i) to[i] = (int)from[i]; /* truncation, as _mm_cvttps_epi32 */
}

ORC_API void orc_vector_convert_int_to_float(const int* from, float* to, int n)
{
	for (int i = 0; i < n; ++i) to[i] = (float)from[i];
}

ORC_API float orc_vector_sum(const float* first, int n)
{
	double s = 0.; /* the reference sums in SSE lanes; any order is within tolerance of the exact sum */
	for (int i = 0; i < n; ++i) s += first[i];
	return (float)s;
}

ORC_API float orc_vector_dot_product(const float* first, const float* second, int n)
{
	double s = 0.;
	for (int i = 0; i < n; ++i) s += (double)first[i] * second[i];
	return (float)s;
}

/* ------------------------------------------------------------------------------------------------------ */
/* broadcasts and reductions */

ORC_API void orc_set_vector_to_matrix_rows(float* result, int h, int w, const float* vec)
{
	for (int r = 0; r < h; ++r) memcpy(result + (size_t)r * w, vec, sizeof(float) * w);
}

ORC_API void orc_add_vector_to_matrix_rows(int batch, const float* m, float* result, int h, int w, const float* vec)
{
	for (int b = 0; b < batch; ++b)
		for (int r = 0; r < h; ++r)
			for (int c = 0; c < w; ++c) {
				const size_t i = ((size_t)b * h + r) * w + c;
				result[i] = m[i] + vec[(size_t)b * w + c];
			}
}

/* sign = +1: AddVectorToMatrixColumns, -1: SubVectorFromMatrixColumns */
ORC_API void orc_add_vector_to_matrix_columns(const float* m, float* result, int h, int w, const float* vec, int sign)
{
	for (int r = 0; r < h; ++r)
		for (int c = 0; c < w; ++c) {
			const size_t i = (size_t)r * w + c;
			result[i] = sign > 0 ? m[i] + vec[r] : m[i] - vec[r];
		}
}

ORC_API void orc_sum_matrix_rows(int batch, float* result, const float* m, int h, int w, int add)
{
	for (int b = 0; b < batch; ++b)
		for (int c = 0; c < w; ++c) {
			float s = 0.f;
			for (int r = 0; r < h; ++r) s += m[((size_t)b * h + r) * w + c];
			if (add) result[(size_t)b * w + c] += s; else result[(size_t)b * w + c] = s;
		}
}

ORC_API void orc_sum_matrix_columns(float* result, const float* m, int h, int w)
{
	for (int r = 0; r < h; ++r) {
		float s = 0.f;
		for (int c = 0; c < w; ++c) s += m[(size_t)r * w + c];
		result[r] = s;
	}
}

ORC_API void orc_multiply_diag_matrix_by_matrix(const float* diag, int n, const float* m, int w, float* result)
{
	for (int r = 0; r < n; ++r)
		for (int c = 0; c < w; ++c) result[(size_t)r * w + c] = diag[r] * m[(size_t)r * w + c];
}

ORC_API void orc_batch_multiply_matrix_by_diag_matrix(int batch, const float* first, int h, int w, int firstOffset,
	const float* second, int secondOffset, float* result)
{
	for (int b = 0; b < batch; ++b)
		for (int r = 0; r < h; ++r)
			for (int c = 0; c < w; ++c)
				result[((size_t)b * h + r) * w + c] =
					first[(size_t)b * firstOffset + (size_t)r * w + c] * second[(size_t)b * secondOffset + c];
}

ORC_API void orc_matrix_softmax_by_rows(const float* m, int h, int w, float* result)
{
	for (int r = 0; r < h; ++r) {
		const float* x = m + (size_t)r * w;
		float* y = result + (size_t)r * w;
		float mx = x[0];
		for (int c = 1; c < w; ++c) if (x[c] > mx) mx = x[c];
		float sum = 0.f;
		for (int c = 0; c < w; ++c) { y[c] = orc_exp_clamped(x[c] - mx); sum += y[c]; }
		const float inv = 1.f / sum;
		for (int c = 0; c < w; ++c) y[c] *= inv;
	}
}

ORC_API void orc_matrix_log_sum_exp_by_rows(const float* m, int h, int w, float* result)
{
	for (int r = 0; r < h; ++r) {
		const float* x = m + (size_t)r * w;
		float mx = x[0];
		for (int c = 1; c < w; ++c) if (x[c] > mx) mx = x[c];
		float sum = 0.f;
		for (int c = 0; c < w; ++c) sum += orc_exp_clamped(x[c] - mx);
		result[r] = mx + logf(sum);
	}
}

ORC_API void orc_find_max_value_in_rows(const float* m, int h, int w, float* result, int* indices)
{
	for (int r = 0; r < h; ++r) {
		const float* x = m + (size_t)r * w;
		int best = 0;
		for (int c = 1; c < w; ++c) if (x[c] > x[best]) best = c;
		result[r] = x[best];
		if (indices) indices[r] = best;
	}
}

ORC_API void orc_find_max_value_in_columns(int batch, const float* m, int h, int w, float* result, int* indices)
{
	for (int b = 0; b < batch; ++b)
		for (int c = 0; c < w; ++c) {
			const float* x = m + (size_t)b * h * w + c;
			int best = 0;
			for (int r = 1; r < h; ++r) if (x[(size_t)r * w] > x[(size_t)best * w]) best = r;
			result[(size_t)b * w + c] = x[(size_t)best * w];
			indices[(size_t)b * w + c] = best;
		}
}

/* [b,h,m,w,c] -> [b,w,m,h,c]; works on 4-byte elements (float and int alike) */
ORC_API void orc_transpose_matrix(int batch, const float* in, int h, int med, int w, int c, float* out)
{
	for (int b = 0; b < batch; ++b)
		for (int j = 0; j < h; ++j)
			for (int m = 0; m < med; ++m)
				for (int i = 0; i < w; ++i)
					for (int ch = 0; ch < c; ++ch)
						out[((((size_t)b * w + i) * med + m) * h + j) * c + ch] =
							in[((((size_t)b * h + j) * med + m) * w + i) * c + ch];
}

/* ------------------------------------------------------------------------------------------------------ */
/* matrix products: row-major, explicit row strides */

/* C[M x N] (+)= A[M x K] * B[N x K]^T */
ORC_API void orc_matmul_nt(const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int add)
{
	for (int i = 0; i < M; ++i)
		for (int j = 0; j < N; ++j) {
			double s = 0.;
			for (int k = 0; k < K; ++k) s += (double)a[(size_t)i * lda + k] * (double)b[(size_t)j * ldb + k];
			if (add) c[(size_t)i * ldc + j] += (float)s; else c[(size_t)i * ldc + j] = (float)s;
		}
}

/* C[M x N] (+)= A[M x K] * B[K x N] */
ORC_API void orc_matmul_nn(const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int add)
{
	for (int i = 0; i < M; ++i)
		for (int j = 0; j < N; ++j) {
			double s = 0.;
			for (int k = 0; k < K; ++k) s += (double)a[(size_t)i * lda + k] * (double)b[(size_t)k * ldb + j];
			if (add) c[(size_t)i * ldc + j] += (float)s; else c[(size_t)i * ldc + j] = (float)s;
		}
}

/* C[M x N] (+)= A[K x M]^T * B[K x N] */
ORC_API void orc_matmul_tn(const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int add)
{
	for (int i = 0; i < M; ++i)
		for (int j = 0; j < N; ++j) {
			double s = 0.;
			for (int k = 0; k < K; ++k) s += (double)a[(size_t)k * lda + i] * (double)b[(size_t)k * ldb + j];
			if (add) c[(size_t)i * ldc + j] += (float)s; else c[(size_t)i * ldc + j] = (float)s;
		}
}

/* ------------------------------------------------------------------------------------------------------ */
/* convolutions and pooling on N,H,W,C images */

ORC_API void orc_conv_output_size(int h, int w, int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw,
	int* ho, int* wo)
{
	*ho = 1 + (h - (fh - 1) * dh + 2 * ph - 1) / sh;
	*wo = 1 + (w - (fw - 1) * dw + 2 * pw - 1) / sw;
}

/* filter [cout][fh][fw][cin]; bias may be null */
ORC_API void orc_blob_convolution(const float* in, int n, int h, int w, int cin, const float* filter, int cout,
	int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw, const float* bias, float* out)
{
	int ho, wo;
	orc_conv_output_size(h, w, fh, fw, ph, pw, sh, sw, dh, dw, &ho, &wo);
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < ho; ++y)
			for (int x = 0; x < wo; ++x)
				for (int co = 0; co < cout; ++co) {
					double s = bias ? bias[co] : 0.;
					for (int ky = 0; ky < fh; ++ky) {
						const int iy = y * sh - ph + ky * dh;
						if (iy < 0 || iy >= h) continue;
						for (int kx = 0; kx < fw; ++kx) {
							const int ix = x * sw - pw + kx * dw;
							if (ix < 0 || ix >= w) continue;
							const float* p = in + (((size_t)b * h + iy) * w + ix) * cin;
							const float* f = filter + (((size_t)co * fh + ky) * fw + kx) * cin;
							for (int ci = 0; ci < cin; ++ci) s += (double)p[ci] * (double)f[ci];
						}
					}
					out[(((size_t)b * ho + y) * wo + x) * cout + co] = (float)s;
				}
}

/* filter [fh][fw][c]; bias may be null; no dilation */
ORC_API void orc_blob_channelwise_convolution(const float* in, int n, int h, int w, int c, const float* filter,
	int fh, int fw, int ph, int pw, int sh, int sw, const float* bias, float* out)
{
	int ho, wo;
	orc_conv_output_size(h, w, fh, fw, ph, pw, sh, sw, 1, 1, &ho, &wo);
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < ho; ++y)
			for (int x = 0; x < wo; ++x)
				for (int ch = 0; ch < c; ++ch) {
					float s = bias ? bias[ch] : 0.f;
					for (int ky = 0; ky < fh; ++ky) {
						const int iy = y * sh - ph + ky;
						if (iy < 0 || iy >= h) continue;
						for (int kx = 0; kx < fw; ++kx) {
							const int ix = x * sw - pw + kx;
							if (ix < 0 || ix >= w) continue;
							s = fmaf(in[(((size_t)b * h + iy) * w + ix) * c + ch], filter[((size_t)ky * fw + kx) * c + ch], s);
						}
					}
					out[(((size_t)b * ho + y) * wo + x) * c + ch] = s;
				}
}

/* Gradient of the convolution by its input, written as the scatter that transposes the forward loop nest: every
 * output pixel sends outputDiff * filter to the input pixels of its window (the definition behind
 * src/CPU/CpuMathEngineDnnConv.cpp:620-805; bias, when given, is a per-channel start value, :758-762). */
ORC_API void orc_blob_convolution_backward(const float* outDiff, int n, int h, int w, int cin, const float* filter, int cout,
	int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw, const float* bias, float* inDiff)
{
	int ho, wo;
	orc_conv_output_size(h, w, fh, fw, ph, pw, sh, sw, dh, dw, &ho, &wo);
	const size_t total = (size_t)n * h * w * cin;
	double* acc = (double*)calloc(total, sizeof(double));
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < ho; ++y)
			for (int x = 0; x < wo; ++x)
				for (int co = 0; co < cout; ++co) {
					const double g = outDiff[(((size_t)b * ho + y) * wo + x) * cout + co];
					for (int ky = 0; ky < fh; ++ky) {
						const int iy = y * sh - ph + ky * dh;
						if (iy < 0 || iy >= h) continue;
						for (int kx = 0; kx < fw; ++kx) {
							const int ix = x * sw - pw + kx * dw;
							if (ix < 0 || ix >= w) continue;
							const float* f = filter + (((size_t)co * fh + ky) * fw + kx) * cin;
							double* dst = acc + (((size_t)b * h + iy) * w + ix) * cin;
							for (int ci = 0; ci < cin; ++ci) dst[ci] += g * f[ci];
						}
					}
				}
	for (size_t i = 0; i < total; ++i) inDiff[i] = (float)(acc[i] + (bias ? bias[i % cin] : 0.f));
	free(acc);
}

/* filterDiff += gradient of the convolution by its filter (src/CPU/CpuMathEngineDnnConv.cpp:808-987) */
ORC_API void orc_blob_convolution_learn_add(const float* in, int n, int h, int w, int cin, const float* outDiff, int cout,
	int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw, float* filterDiff)
{
	int ho, wo;
	orc_conv_output_size(h, w, fh, fw, ph, pw, sh, sw, dh, dw, &ho, &wo);
	for (int co = 0; co < cout; ++co)
		for (int ky = 0; ky < fh; ++ky)
			for (int kx = 0; kx < fw; ++kx)
				for (int ci = 0; ci < cin; ++ci) {
					double s = 0;
					for (int b = 0; b < n; ++b)
						for (int y = 0; y < ho; ++y) {
							const int iy = y * sh - ph + ky * dh;
							if (iy < 0 || iy >= h) continue;
							for (int x = 0; x < wo; ++x) {
								const int ix = x * sw - pw + kx * dw;
								if (ix < 0 || ix >= w) continue;
								s += (double)outDiff[(((size_t)b * ho + y) * wo + x) * cout + co]
									* in[(((size_t)b * h + iy) * w + ix) * cin + ci];
							}
						}
					float* d = filterDiff + (((size_t)co * fh + ky) * fw + kx) * cin + ci;
					*d = (float)(*d + s);
				}
}

/* result[r] = <first[r], second[r]> (src/CPU/CpuMathEngineBlas.cpp RowMultiplyMatrixByMatrix) */
ORC_API void orc_row_multiply_matrix_by_matrix(const float* first, const float* second, int h, int w, float* result)
{
	for (int r = 0; r < h; ++r) {
		double s = 0;
		for (int c = 0; c < w; ++c) s += (double)first[(size_t)r * w + c] * second[(size_t)r * w + c];
		result[r] = (float)s;
	}
}

/* dE/dx of a softmax over rows from its output y = first and dE/dy = second: y * ( dE/dy - <dE/dy, y> )
 * (src/CPU/CpuMathEngineBlas.cpp:1161-1179) */
ORC_API void orc_matrix_softmax_diff_op_by_rows(const float* first, const float* second, int h, int w, float* result)
{
	for (int r = 0; r < h; ++r) {
		double dot = 0;
		for (int c = 0; c < w; ++c) dot += (double)first[(size_t)r * w + c] * second[(size_t)r * w + c];
		for (int c = 0; c < w; ++c)
			result[(size_t)r * w + c] = first[(size_t)r * w + c] * (second[(size_t)r * w + c] - (float)dot);
	}
}

/* result[j][c] += sum over b of first[b][j] * second[b][j][c] (src/CPU/x86/CpuX86MathEngineBlas.cpp:401-456) */
ORC_API void orc_multiply_diag_matrix_by_matrix_and_add(int batch, const float* first, int size, const float* second, int width,
	float* result)
{
	for (int j = 0; j < size; ++j)
		for (int c = 0; c < width; ++c) {
			double s = result[(size_t)j * width + c];
			for (int b = 0; b < batch; ++b)
				s += (double)first[(size_t)b * size + j] * second[((size_t)b * size + j) * width + c];
			result[(size_t)j * width + c] = (float)s;
		}
}

/* Dropout as the reference's CPU engine draws it (src/CPU/CpuMathEngineDnnDropout.cpp:33-96, generator src/CPU/CpuRandom.h):
 * ten rounds of Philox 4x32 on a running 128-bit counter, four mask values per counter value, consumed in the loop
 * order of the engine (mask chunks of 64 values; spatial: object after object of the batch width). */
typedef struct { unsigned seed; unsigned counter[4]; } orc_random;

static void orc_random_next(orc_random* r, unsigned out[4])
{
	unsigned key[2] = { r->seed, r->seed ^ 0xBADF00Du };
	unsigned c[4] = { r->counter[0], r->counter[1], r->counter[2], r->counter[3] };
	for (int round = 0; round < 10; ++round) {
		const unsigned long long first = 0xD2511F53ull * c[0];
		const unsigned long long second = 0xCD9E8D57ull * c[2];
		const unsigned n0 = (unsigned)(second >> 32) ^ c[1] ^ key[0];
		const unsigned n2 = (unsigned)(first >> 32) ^ c[3] ^ key[1];
		c[1] = (unsigned)second; c[3] = (unsigned)first; c[0] = n0; c[2] = n2;
		key[0] += 0x9E3779B9u;
		key[1] += 0xBB67AE85u;
	}
	for (int k = 0; k < 4; ++k) out[k] = c[k];
	if (++r->counter[0] == 0 && ++r->counter[1] == 0 && ++r->counter[2] == 0) ++r->counter[3];
}

/* dims: the 7 blob dimensions */
ORC_API void orc_dropout(const int* dims, float rate, int isSpatial, int isBatchwise, int seed, const float* in, float* out)
{
	const float forwardRate = 1.f - rate;
	const int objectCount = dims[0] * dims[1] * dims[2];
	const int inputObjectSize = dims[3] * dims[4] * dims[5] * dims[6];
	if (forwardRate == 1.f) {
		memcpy(out, in, sizeof(float) * (size_t)objectCount * inputObjectSize);
		return;
	}
	const float value = 1.f / forwardRate;
	const unsigned threshold = (unsigned)((double)forwardRate * 4294967295.0);
	const int objectSize = isSpatial ? dims[6] : inputObjectSize;
	const int batchLength = isBatchwise ? objectCount : dims[0];
	const int batchWidth = objectCount / batchLength;
	const int unitSize = isSpatial ? objectSize : batchWidth * objectSize;
	const int pixels = isSpatial ? inputObjectSize / objectSize : 1;
	const int objects = isSpatial ? batchWidth : 1;
	const size_t sliceStep = isSpatial ? (size_t)batchWidth * inputObjectSize : (size_t)unitSize;
	orc_random random = { (unsigned)seed, { 0, 0, (unsigned)seed ^ 0xBADFACEu, (unsigned)seed ^ 0xBADBEEFu } };
	float mask[64];
	for (int object = 0; object < objects; ++object) {
		const size_t base = isSpatial ? (size_t)object * inputObjectSize : 0;
		for (int chunk = 0; chunk * 64 < unitSize; ++chunk) {
			const int size = unitSize - chunk * 64 < 64 ? unitSize - chunk * 64 : 64;
			for (int g = 0; g * 4 < size; ++g) {
				unsigned word[4];
				orc_random_next(&random, word);
				for (int k = 0; k < 4; ++k) mask[g * 4 + k] = word[k] <= threshold ? value : 0.f;
			}
			for (int b = 0; b < batchLength; ++b)
				for (int p = 0; p < pixels; ++p) {
					const size_t at = base + b * sliceStep + (size_t)p * objectSize + (size_t)chunk * 64;
					for (int k = 0; k < size; ++k) out[at + k] = in[at + k] * mask[k];
				}
		}
	}
}

/* BroadcastCopy: `from` repeats along every dimension where it has size 1 and `to` does not; width is one more,
 * innermost, dimension that both share (src/CPU/CpuMathEngineVectorMath.cpp:69-95 builds the same result by growing
 * the copied block dimension by dimension from the innermost) */
ORC_API void orc_broadcast_copy(const int* toDims, const int* fromDims, int width, const float* from, float* to)
{
	size_t fromStride[7];
	size_t stride = (size_t)width, total = (size_t)width;
	for (int d = 6; d >= 0; --d) {
		fromStride[d] = fromDims[d] == toDims[d] ? stride : 0;
		stride *= (size_t)fromDims[d];
		total *= (size_t)toDims[d];
	}
	for (size_t i = 0; i < total; ++i) {
		size_t rest = i / (size_t)width, source = i % (size_t)width;
		for (int d = 6; d >= 0; --d) {
			source += (rest % (size_t)toDims[d]) * fromStride[d];
			rest /= (size_t)toDims[d];
		}
		to[i] = from[source];
	}
}

/* Gradients of the channelwise convolution, as the transposes of its forward loop nest
 * (src/CPU/CpuMathEngineDnnConv.cpp:1017-1200): by the input (scatter of outputDiff * filter), by the filter
 * and by the free term (sums over the pixels, added to what the buffers hold) */
ORC_API void orc_blob_channelwise_convolution_backward(const float* outDiff, int n, int h, int w, int c, const float* filter,
	int fh, int fw, int ph, int pw, int sh, int sw, float* inDiff)
{
	const int ho = (h + 2 * ph - fh) / sh + 1, wo = (w + 2 * pw - fw) / sw + 1;
	const size_t total = (size_t)n * h * w * c;
	double* acc = (double*)calloc(total, sizeof(double));
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < ho; ++y)
			for (int x = 0; x < wo; ++x)
				for (int ky = 0; ky < fh; ++ky) {
					const int iy = y * sh - ph + ky;
					if (iy < 0 || iy >= h) continue;
					for (int kx = 0; kx < fw; ++kx) {
						const int ix = x * sw - pw + kx;
						if (ix < 0 || ix >= w) continue;
						for (int ch = 0; ch < c; ++ch)
							acc[(((size_t)b * h + iy) * w + ix) * c + ch] +=
								(double)outDiff[(((size_t)b * ho + y) * wo + x) * c + ch] * filter[((size_t)ky * fw + kx) * c + ch];
					}
				}
	for (size_t i = 0; i < total; ++i) inDiff[i] = (float)acc[i];
	free(acc);
}

ORC_API void orc_blob_channelwise_convolution_learn_add(const float* in, int n, int h, int w, int c, const float* outDiff,
	int fh, int fw, int ph, int pw, int sh, int sw, float* filterDiff, float* freeTermDiff)
{
	const int ho = (h + 2 * ph - fh) / sh + 1, wo = (w + 2 * pw - fw) / sw + 1;
	for (int ch = 0; ch < c; ++ch) {
		for (int ky = 0; ky < fh; ++ky)
			for (int kx = 0; kx < fw; ++kx) {
				double s = 0;
				for (int b = 0; b < n; ++b)
					for (int y = 0; y < ho; ++y) {
						const int iy = y * sh - ph + ky;
						if (iy < 0 || iy >= h) continue;
						for (int x = 0; x < wo; ++x) {
							const int ix = x * sw - pw + kx;
							if (ix < 0 || ix >= w) continue;
							s += (double)outDiff[(((size_t)b * ho + y) * wo + x) * c + ch] * in[(((size_t)b * h + iy) * w + ix) * c + ch];
						}
					}
				float* d = filterDiff + ((size_t)ky * fw + kx) * c + ch;
				*d = (float)(*d + s);
			}
		if (freeTermDiff) {
			double s = 0;
			for (size_t p = 0; p < (size_t)n * ho * wo; ++p) s += outDiff[p * c + ch];
			freeTermDiff[ch] = (float)(freeTermDiff[ch] + s);
		}
	}
}

/* sourceDiff = 0, then every output element adds its gradient at the index the forward pass stored
 * (src/CPU/CpuMathEngineDnnPooling.cpp:146-175) */
ORC_API void orc_blob_max_pooling_backward(const float* resultDiff, const int* indices, int n, int sourceObjectSize,
	int resultObjectSize, float* sourceDiff)
{
	memset(sourceDiff, 0, (size_t)n * sourceObjectSize * sizeof(float));
	for (int b = 0; b < n; ++b)
		for (int j = 0; j < resultObjectSize; ++j)
			sourceDiff[(size_t)b * sourceObjectSize + indices[(size_t)b * resultObjectSize + j]] += resultDiff[(size_t)b * resultObjectSize + j];
}

/* every window spreads its gradient over its elements, the sums are scaled by 1 / fh / fw at the end
 * (src/CPU/CpuMathEngineDnnPooling.cpp:202-242) */
ORC_API void orc_blob_mean_pooling_backward(const float* resultDiff, int n, int h, int w, int c, int fh, int fw, int sh, int sw,
	float* sourceDiff)
{
	const int ho = (h - fh) / sh + 1, wo = (w - fw) / sw + 1;
	memset(sourceDiff, 0, (size_t)n * h * w * c * sizeof(float));
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < ho; ++y)
			for (int x = 0; x < wo; ++x)
				for (int ky = 0; ky < fh; ++ky)
					for (int kx = 0; kx < fw; ++kx)
						for (int ch = 0; ch < c; ++ch)
							sourceDiff[(((size_t)b * h + y * sh + ky) * w + x * sw + kx) * c + ch]
								+= resultDiff[(((size_t)b * ho + y) * wo + x) * c + ch];
	const float scale = 1.f / fh / fw;
	for (size_t i = 0; i < (size_t)n * h * w * c; ++i) sourceDiff[i] *= scale;
}

/* Max pooling without padding. indices may be null. The index follows the reference CPU engine literally:
 * strip maxima over the window rows per image column (topmost row on ties), window maximum over the fw column
 * maxima (leftmost on ties), and the row is read from the strip's row-index buffer at position
 * columnIndex * channels + c, i.e. relative to the window start, NOT offset by the window's column. */
ORC_API void orc_blob_max_pooling(const float* in, int n, int h, int w, int c, int fh, int fw, int sh, int sw,
	int* indices, float* out)
{
	const int ho = (h - fh) / sh + 1, wo = (w - fw) / sw + 1;
	const int rowSize = w * c;
	float* colMax = (float*)malloc(sizeof(float) * rowSize);
	int* rowIdx = (int*)malloc(sizeof(int) * rowSize);
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < ho; ++y) {
			const int stripRow = y * sh;
			const float* strip = in + ((size_t)b * h + stripRow) * rowSize;
			for (int i = 0; i < rowSize; ++i) { colMax[i] = strip[i]; rowIdx[i] = 0; }
			for (int ky = 1; ky < fh; ++ky)
				for (int i = 0; i < rowSize; ++i)
					if (strip[(size_t)ky * rowSize + i] > colMax[i]) { colMax[i] = strip[(size_t)ky * rowSize + i]; rowIdx[i] = ky; }
			for (int x = 0; x < wo; ++x) {
				const int windowColumn = x * sw * c;
				for (int ch = 0; ch < c; ++ch) {
					float best = colMax[windowColumn + ch];
					int bestCol = 0;
					for (int kx = 1; kx < fw; ++kx)
						if (colMax[windowColumn + kx * c + ch] > best) { best = colMax[windowColumn + kx * c + ch]; bestCol = kx; }
					const size_t o = (((size_t)b * ho + y) * wo + x) * c + ch;
					out[o] = best;
					if (indices) {
						const int windowIndex = bestCol * c + ch;
						indices[o] = (stripRow + rowIdx[windowIndex]) * rowSize + windowColumn + windowIndex;
					}
				}
			}
		}
	free(colMax);
	free(rowIdx);
}

ORC_API void orc_blob_mean_pooling(const float* in, int n, int h, int w, int c, int fh, int fw, int sh, int sw, float* out)
{
	const int ho = (h - fh) / sh + 1, wo = (w - fw) / sw + 1;
	const float scale = 1.f / fh / fw;
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < ho; ++y)
			for (int x = 0; x < wo; ++x)
				for (int ch = 0; ch < c; ++ch) {
					float s = 0.f;
					for (int kx = 0; kx < fw; ++kx) {
						float col = 0.f;
						for (int ky = 0; ky < fh; ++ky) {
							const float v = in[(((size_t)b * h + y * sh + ky) * w + x * sw + kx) * c + ch];
							col = ky == 0 ? v : col + v;
						}
						s = kx == 0 ? col : s + col;
					}
					out[(((size_t)b * ho + y) * wo + x) * c + ch] = s * scale;
				}
}

/* ------------------------------------------------------------------------------------------------------ */
/* data movement */

static int orc_resize_coord(int x, int size, int padding)
{
	if (x >= 0 && x < size) return x;
	if (padding == 0) return -1;
	if (padding == 1) return x < 0 ? 0 : size - 1;
	return x < 0 ? -(x % size) : (2 * size - 2 - (x % size)) % size;
}

/* padding: 0 constant, 1 edge, 2 reflect; negative deltas crop */
ORC_API void orc_blob_resize_image(const float* from, int n, int h, int w, int c, int dl, int dr, int dt, int db,
	int padding, float value, float* to)
{
	const int th = h + dt + db, tw = w + dl + dr;
	for (int b = 0; b < n; ++b)
		for (int y = 0; y < th; ++y)
			for (int x = 0; x < tw; ++x) {
				const int sy = orc_resize_coord(y - dt, h, padding), sx = orc_resize_coord(x - dl, w, padding);
				const int inside = sy >= 0 && sy < h && sx >= 0 && sx < w;
				for (int ch = 0; ch < c; ++ch)
					to[(((size_t)b * th + y) * tw + x) * c + ch] = inside ? from[(((size_t)b * h + sy) * w + sx) * c + ch] : value;
			}
}

/* big blob = [rows][rowSize]; part i = [rows][sizes[i]] holding columns [sum sizes[<i], ...) of every row.
 * merge != 0 copies parts -> big, else big -> parts. (dim == 0 is rows = 1, sizes = whole blob sizes.) */
ORC_API void orc_blob_split_merge(float* big, int rows, float* const* parts, const int* sizes, int count, int merge)
{
	int rowSize = 0;
	for (int i = 0; i < count; ++i) rowSize += sizes[i];
	for (int r = 0; r < rows; ++r) {
		int off = 0;
		for (int i = 0; i < count; ++i) {
			float* small = parts[i] + (size_t)r * sizes[i];
			float* large = big + (size_t)r * rowSize + off;
			if (merge) memcpy(large, small, sizeof(float) * sizes[i]); else memcpy(small, large, sizeof(float) * sizes[i]);
			off += sizes[i];
		}
	}
}

/* ------------------------------------------------------------------------------------------------------ */
/* LSTM: inputWeights [4H x In], recurrentWeights [4H x H], gates main | forget | input | output.
 * free terms, initial state c0 / output h0 and the state output may be null. x: [T][B][In], h, c: [T][B][H]. */
ORC_API void orc_lstm(int H, int In, const float* wIn, const float* bIn, const float* wRec, const float* bRec,
	int reverse, int T, int B, const float* c0, const float* h0, const float* x, float* cOut, float* hOut)
{
	float* gates = (float*)malloc(sizeof(float) * 4 * H);
	float* cPrev = (float*)calloc((size_t)B * H, sizeof(float));
	float* hPrev = (float*)calloc((size_t)B * H, sizeof(float));
	if (c0) memcpy(cPrev, c0, sizeof(float) * B * H);
	if (h0) memcpy(hPrev, h0, sizeof(float) * B * H);
	for (int i = 0; i < T; ++i) {
		const int t = reverse ? T - 1 - i : i;
		for (int b = 0; b < B; ++b) {
			const float* xt = x + ((size_t)t * B + b) * In;
			for (int g = 0; g < 4 * H; ++g) {
				double s = 0.;
				for (int k = 0; k < In; ++k) s += (double)xt[k] * (double)wIn[(size_t)g * In + k];
				for (int k = 0; k < H; ++k) s += (double)hPrev[(size_t)b * H + k] * (double)wRec[(size_t)g * H + k];
				if (bIn && bRec) s += bIn[g] + bRec[g];
				else if (bIn) s += bIn[g];
				else if (bRec) s += bRec[g];
				gates[g] = (float)s;
			}
			for (int j = 0; j < H; ++j) {
				float a, f, in, o;
				orc_vector_unary(ORC_TANH, gates + j, &a, 1, 0, 0);
				orc_vector_unary(ORC_SIGMOID, gates + H + j, &f, 1, 0, 0);
				orc_vector_unary(ORC_SIGMOID, gates + 2 * H + j, &in, 1, 0, 0);
				orc_vector_unary(ORC_SIGMOID, gates + 3 * H + j, &o, 1, 0, 0);
				const float c = f * cPrev[(size_t)b * H + j] + in * a;
				float tc;
				orc_vector_unary(ORC_TANH, &c, &tc, 1, 0, 0);
				if (cOut) cOut[((size_t)t * B + b) * H + j] = c;
				hOut[((size_t)t * B + b) * H + j] = o * tc;
				gates[j] = c; /* new state, copied back below */
			}
			for (int j = 0; j < H; ++j) cPrev[(size_t)b * H + j] = gates[j];
		}
		memcpy(hPrev, hOut + (size_t)t * B * H, sizeof(float) * B * H);
	}
	free(gates);
	free(cPrev);
	free(hPrev);
}

/* CTC greedy collapse: labels [B][T] (arg-max per step, sequence-major as the decoding layer stores them after
 * its transpose) -> per sequence the labels that differ from blank and from the previous step; out [B][T],
 * lengths [B]. seqLen may be null (= T for every sequence). */
ORC_API void orc_ctc_greedy_collapse(const int* labels, int T, int B, int blank, const int* seqLen, int* out, int* lengths)
{
	for (int b = 0; b < B; ++b) {
		const int len = seqLen ? seqLen[b] : T;
		int n = 0;
		for (int t = 0; t < len; ++t) {
			const int l = labels[(size_t)b * T + t];
			if (l != blank && (t == 0 || l != labels[(size_t)b * T + t - 1])) out[(size_t)b * T + n++] = l;
		}
		lengths[b] = n;
	}
}
