/* TEST INFRASTRUCTURE ONLY — see lten_oracle.h.  Plain C, no vector intrinsics, built
 * with -O2 -ffp-contract=off so that every fp32 operation below is a single IEEE
 * operation in the order written. */
#include "lten_oracle.h"

#include <limits.h>
#include <pthread.h>
#include <stdlib.h>
#include <math.h>
#include <string.h>

#define ORACLE_MAX_DIMS 16 /* l-ten/md_array.h:37 */

/* ------------------------------------------------------------------ requantize */

float oracle_real_multiplier(float scale_a, float scale_b, float scale_c)
{
	/* l-ten/math_fns.cpp:1436 */
	volatile float ab = scale_a * scale_b;
	return ab / scale_c;
}

uint8_t oracle_requantize(float real_multiplier, int32_t element, uint8_t zero_point)
{
	/* l-ten/math_fns.cpp:1474.  The C++ cast float -> unsigned char is undefined
	 * outside [0,255]; l-ten's build (g++ -O2, x86-64) lowers it to cvttss2si and a
	 * byte store, which is what is spelled out here. */
	volatile float f = (float)element;
	volatile float p = real_multiplier * f;
	volatile float s = p + (float)zero_point;
	float v = s;
	int32_t i;
	if (v >= -2147483648.0f && v < 2147483648.0f)
		i = (int32_t)v;
	else
		i = INT32_MIN; /* NaN, +-Inf, |v| >= 2^31 */
	return (uint8_t)((uint32_t)i & 0xFFu);
}

/* ------------------------------------------------------------ quantized_matmul */

int oracle_quantized_matmul(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, uint8_t alpha,
                            const uint8_t* A, const uint8_t* B, uint8_t beta, uint8_t* C,
                            const oracle_qparams* qp, const int32_t* bias, int32_t* workspace,
                            int32_t* acc_out)
{
	uint64_t i, j, k;
	int32_t* row_vector = workspace;     /* l-ten/math_fns.cpp:1325 */
	int32_t* col_vector = workspace + N; /* :1326 */
	const int32_t zpA = qp[0].zero_point;
	const int32_t zpB = qp[1].zero_point;

	if (alpha != 1 || beta != 0) /* :1331 */
		return -1;

	/* :1336-1429 — sums over K of every B "row" j and every A "row" i, in the
	 * storage order selected by the transpose flags, times the other zero point. */
	for (j = 0; j < N; j++) {
		uint32_t s = 0;
		for (k = 0; k < K; k++)
			s += tB ? B[j * K + k] : B[k * N + j];
		row_vector[j] = (int32_t)(s * (uint32_t)(-zpA));
	}
	for (i = 0; i < M; i++) {
		uint32_t s = 0;
		for (k = 0; k < K; k++)
			s += tA ? A[k * M + i] : A[i * K + k];
		col_vector[i] = (int32_t)(s * (uint32_t)(-zpB));
	}

	/* :1433 */
	const uint64_t broadcast_val = K * (uint64_t)zpA * (uint64_t)zpB;
	/* :1436 */
	const float real_multiplier = oracle_real_multiplier(qp[0].scale, qp[1].scale, qp[2].scale);

	/* :1438-1476.  Unsigned arithmetic so that wrap-around is defined; equal to the
	 * reference's int arithmetic wherever that does not overflow. */
	for (i = 0; i < M; i++) {
		for (j = 0; j < N; j++) {
			uint32_t e = 0;
			if (!tA && tB) {
				const uint8_t* a = A + i * K;
				const uint8_t* b = B + j * K;
				for (k = 0; k < K; k++)
					e += (uint32_t)a[k] * b[k];
			} else if (!tA && !tB) {
				for (k = 0; k < K; k++)
					e += (uint32_t)A[i * K + k] * B[j + N * k];
			} else if (tA && !tB) {
				for (k = 0; k < K; k++)
					e += (uint32_t)A[k * M + i] * B[j + N * k];
			} else {
				for (k = 0; k < K; k++)
					e += (uint32_t)A[k * M + i] * B[j * K + k];
			}
			e += (uint32_t)row_vector[j] + (uint32_t)col_vector[i] + (uint32_t)broadcast_val; /* :1469 */
			if (bias)
				e += (uint32_t)bias[j]; /* :1472 */
			if (acc_out)
				acc_out[i * N + j] = (int32_t)e;
			C[i * N + j] = oracle_requantize(real_multiplier, (int32_t)e, qp[2].zero_point); /* :1474 */
		}
	}
	return 0;
}

/* ----------------------------------------------------------------------- sgemm */

static void sgemm_rows(int tA, int tB, uint64_t m0, uint64_t m1, uint64_t N, uint64_t K, float alpha,
                       const float* A, uint64_t lda, const float* B, uint64_t ldb, float beta,
                       float* C, uint64_t ldc)
{
	uint64_t m, n, k;
	for (m = m0; m < m1; m++) {
		float* c = C + m * ldc;
		/* l-ten/math_fns.cpp:1221-1234: beta == 0 overwrites, otherwise scales. */
		if (beta == 0.0f)
			for (n = 0; n < N; n++) c[n] = 0.0f;
		else
			for (n = 0; n < N; n++) c[n] = c[n] * beta;
		if (!tB) {
			/* For a fixed (m, n) the terms arrive in increasing k, as in
			 * l-ten/math_fns.cpp:822-831 (NN) and :794-803 (TN). */
			for (k = 0; k < K; k++) {
				float a = tA ? A[k * lda + m] : A[m * lda + k];
				if (alpha != 1.0f) a = a * alpha; /* :1236-1242 */
				const float* b = B + k * ldb;
				for (n = 0; n < N; n++) c[n] += a * b[n];
			}
		} else {
			/* l-ten/math_fns.cpp:809-818 (NT) and :779-788 (TT) */
			for (n = 0; n < N; n++) {
				const float* b = B + n * ldb;
				float acc = c[n];
				for (k = 0; k < K; k++) {
					float a = tA ? A[k * lda + m] : A[m * lda + k];
					if (alpha != 1.0f) a = a * alpha;
					acc += a * b[k];
				}
				c[n] = acc;
			}
		}
	}
}

void oracle_sgemm(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, float alpha, const float* A,
                  uint64_t lda, const float* B, uint64_t ldb, float beta, float* C, uint64_t ldc)
{
	sgemm_rows(tA, tB, 0, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}

void oracle_sgemm_f64(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, float alpha, const float* A,
                      uint64_t lda, const float* B, uint64_t ldb, float beta, float* C, uint64_t ldc)
{
	uint64_t m, n, k;
	double* acc = (double*)malloc(sizeof(double) * (N ? N : 1));
	for (m = 0; m < M; m++) {
		for (n = 0; n < N; n++) acc[n] = 0.0;
		for (k = 0; k < K; k++) {
			double a = tA ? A[k * lda + m] : A[m * lda + k];
			if (!tB) {
				const float* b = B + k * ldb;
				for (n = 0; n < N; n++) acc[n] += a * (double)b[n];
			} else {
				for (n = 0; n < N; n++) acc[n] += a * (double)B[n * ldb + k];
			}
		}
		for (n = 0; n < N; n++) {
			double c0 = (beta == 0.0f) ? 0.0 : (double)beta * (double)C[m * ldc + n];
			C[m * ldc + n] = (float)((double)alpha * acc[n] + c0);
		}
	}
	free(acc);
}

typedef struct {
	int tA, tB;
	uint64_t M, N, K;
	float alpha, beta;
	const float *A, *B;
	float* C;
	uint64_t lda, ldb, ldc;
	int index, total;
} mt_job;

static void* mt_worker(void* p)
{
	mt_job* j = (mt_job*)p;
	/* l-ten/math_fns.cpp:1128: 4-row blocks, block b goes to worker b % total. */
	uint64_t m;
	for (m = (uint64_t)j->index * 4; m < j->M; m += 4 * (uint64_t)j->total) {
		uint64_t m1 = m + 4 < j->M ? m + 4 : j->M;
		sgemm_rows(j->tA, j->tB, m, m1, j->N, j->K, j->alpha, j->A, j->lda, j->B, j->ldb, j->beta, j->C, j->ldc);
	}
	return NULL;
}

void oracle_sgemm_mt(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, float alpha, const float* A,
                     uint64_t lda, const float* B, uint64_t ldb, float beta, float* C, uint64_t ldc,
                     int threads)
{
	if (threads < 1) threads = 1;
	if (threads > 256) threads = 256;
	if (M <= 4 || threads == 1) { /* l-ten/math_fns.cpp:1270 */
		sgemm_rows(tA, tB, 0, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
		return;
	}
	pthread_t tid[256];
	mt_job job[256];
	int t;
	for (t = 0; t < threads; t++) {
		mt_job j = { tA, tB, M, N, K, alpha, beta, A, B, C, lda, ldb, ldc, t, threads };
		job[t] = j;
		pthread_create(&tid[t], NULL, mt_worker, &job[t]);
	}
	for (t = 0; t < threads; t++) pthread_join(tid[t], NULL);
}

/* --------------------------------------------------------------- im2col/col2im */

#define IM2COL_BODY(T)                                                                           \
	uint64_t Ho = (H + 2 * ph - kh) / sh + 1;                                                \
	uint64_t Wo = (W + 2 * pw - kw) / sw + 1;                                                \
	uint64_t Ccol = C * kh * kw;                                                             \
	uint64_t c, h, w;                                                                        \
	for (c = 0; c < Ccol; c++) {                                                             \
		uint64_t wo = c % kw, ho = (c / kw) % kh, ci = c / kh / kw;                      \
		for (h = 0; h < Ho; h++)                                                         \
			for (w = 0; w < Wo; w++) {                                               \
				/* l-ten/im_col.h:22-23: unsigned wrap-around stands in for "negative" */ \
				uint64_t hp = h * sh - ph + ho, wp = w * sw - pw + wo;           \
				col[(c * Ho + h) * Wo + w] = (hp < H && wp < W) ? im[(ci * H + hp) * W + wp] : (T)0; \
			}                                                                        \
	}

void oracle_im2col_f32(const float* im, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                       uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, float* col)
{
	IM2COL_BODY(float)
}

void oracle_im2col_u8(const uint8_t* im, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                      uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, uint8_t* col)
{
	IM2COL_BODY(uint8_t)
}

void oracle_col2im_f32(const float* col, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                       uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, float* im)
{
	/* l-ten/im_col.h:35-57: scatter-add, caller zeroes `im`. */
	uint64_t Ho = (H + 2 * ph - kh) / sh + 1;
	uint64_t Wo = (W + 2 * pw - kw) / sw + 1;
	uint64_t Ccol = C * kh * kw;
	uint64_t c, h, w;
	for (c = 0; c < Ccol; c++) {
		uint64_t wo = c % kw, ho = (c / kw) % kh, ci = c / kh / kw;
		for (h = 0; h < Ho; h++)
			for (w = 0; w < Wo; w++) {
				uint64_t hp = h * sh - ph + ho, wp = w * sw - pw + wo;
				if (hp < H && wp < W)
					im[(ci * H + hp) * W + wp] += col[(c * Ho + h) * Wo + w];
			}
	}
}

/* ------------------------------------------------------------- FullyConnected */

void oracle_fc_forward(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W,
                       const float* bias, float* Y)
{
	uint64_t m;
	/* l-ten/fully_connected.cpp:113 */
	oracle_sgemm(0, 1, M, out, in, 1.0f, X, in, W, in, 0.0f, Y, out);
	if (bias) {
		/* :115-123 — ones[M x 1] * bias[1 x out] added with beta = 1 */
		float* ones = (float*)malloc(sizeof(float) * (M ? M : 1));
		for (m = 0; m < M; m++) ones[m] = 1.0f;
		oracle_sgemm(0, 0, M, out, 1, 1.0f, ones, 1, bias, out, 1.0f, Y, out);
		free(ones);
	}
}

void oracle_fc_backward(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W,
                        const float* dY, float* dX, float* dW, float* db_accum)
{
	uint64_t m;
	if (dX) /* l-ten/backprop.cpp:2151 */
		oracle_sgemm(0, 0, M, in, out, 1.0f, dY, out, W, in, 0.0f, dX, in);
	if (dW) /* :2167 */
		oracle_sgemm(1, 0, out, in, M, 1.0f, dY, out, X, in, 0.0f, dW, in);
	if (db_accum) { /* :2170-2183 */
		float* ones = (float*)malloc(sizeof(float) * (M ? M : 1));
		for (m = 0; m < M; m++) ones[m] = 1.0f;
		oracle_sgemm(0, 0, 1, out, M, 1.0f, ones, M, dY, out, 1.0f, db_accum, out);
		free(ones);
	}
}

int oracle_fcq_forward(uint64_t batch, uint64_t M, uint64_t in, uint64_t out, const uint8_t* X,
                       const uint8_t* W, const int32_t* bias, const oracle_qparams* qp, uint8_t* Y)
{
	/* l-ten/fully_connected.cpp:364-396: one quantized_matmul(false, true, ...) per leading index. */
	int32_t* ws = (int32_t*)malloc(sizeof(int32_t) * (M + out + 1));
	uint64_t b;
	int rc = 0;
	for (b = 0; b < batch && rc == 0; b++)
		rc = oracle_quantized_matmul(0, 1, M, out, in, 1, X + b * M * in, W, 0, Y + b * M * out, qp, bias, ws, NULL);
	free(ws);
	return rc;
}

/* --------------------------------------------------------------------- matmul */

static uint64_t bcast_offset(const uint64_t* coord, const uint64_t* dims, const uint64_t* strides, int n)
{
	/* l-ten/md_array.h:1258-1269: coordinate clamped to dim-1 */
	uint64_t off = 0;
	int i;
	for (i = 0; i < n; i++) {
		uint64_t c = coord[i] < dims[i] - 1 ? coord[i] : dims[i] - 1;
		off += c * strides[i];
	}
	return off;
}

static void row_major_strides(int ndims, const uint64_t* dims, uint64_t* strides)
{
	int i;
	uint64_t s = 1;
	for (i = ndims - 1; i >= 0; i--) {
		strides[i] = s;
		s *= dims[i];
	}
}

static int matmul_shapes(int ndims, const uint64_t* adims, const uint64_t* bdims, uint64_t* cdims)
{
	int i;
	if (ndims < 3 || ndims > ORACLE_MAX_DIMS) return -1;
	if (adims[ndims - 1] != bdims[ndims - 2]) return -1; /* l-ten/md_array.h:985 */
	for (i = 0; i < ndims - 2; i++) {                    /* :1230-1246 */
		if (adims[i] != bdims[i] && adims[i] != 1 && bdims[i] != 1) return -1;
		cdims[i] = adims[i] > bdims[i] ? adims[i] : bdims[i];
	}
	cdims[ndims - 2] = adims[ndims - 2];
	cdims[ndims - 1] = bdims[ndims - 1];
	return 0;
}

static int next_index(uint64_t* idx, const uint64_t* dims, int n)
{
	int i;
	for (i = n - 1; i >= 0; i--) {
		if (++idx[i] < dims[i]) return 1;
		idx[i] = 0;
	}
	return 0;
}

int oracle_matmul(int ndims, const uint64_t* adims, const uint64_t* bdims, const float* A,
                  const float* B, uint64_t* cdims, float* C)
{
	uint64_t sa[ORACLE_MAX_DIMS], sb[ORACLE_MAX_DIMS], sc[ORACLE_MAX_DIMS], idx[ORACLE_MAX_DIMS] = { 0 };
	if (matmul_shapes(ndims, adims, bdims, cdims)) return -1;
	row_major_strides(ndims, adims, sa);
	row_major_strides(ndims, bdims, sb);
	row_major_strides(ndims, cdims, sc);
	uint64_t M = cdims[ndims - 2], N = cdims[ndims - 1], K = adims[ndims - 1];
	uint64_t total = 1;
	int i;
	for (i = 0; i < ndims - 2; i++) total *= cdims[i];
	if (total == 0) return 0;
	do { /* l-ten/md_array.h:1000-1007 */
		oracle_sgemm(0, 0, M, N, K, 1.0f, A + bcast_offset(idx, adims, sa, ndims - 2), K,
		             B + bcast_offset(idx, bdims, sb, ndims - 2), N, 0.0f,
		             C + bcast_offset(idx, cdims, sc, ndims - 2), N);
	} while (next_index(idx, cdims, ndims - 2));
	return 0;
}

int oracle_matmul_backward(int ndims, const uint64_t* adims, const uint64_t* bdims, const float* A,
                           const float* B, const float* dC, float* dA, float* dB)
{
	uint64_t cdims[ORACLE_MAX_DIMS], sa[ORACLE_MAX_DIMS], sb[ORACLE_MAX_DIMS], sc[ORACLE_MAX_DIMS];
	uint64_t idx[ORACLE_MAX_DIMS] = { 0 };
	if (matmul_shapes(ndims, adims, bdims, cdims)) return -1;
	row_major_strides(ndims, adims, sa);
	row_major_strides(ndims, bdims, sb);
	row_major_strides(ndims, cdims, sc);
	uint64_t M = cdims[ndims - 2], N = cdims[ndims - 1], K = adims[ndims - 1];
	uint64_t na = 1, nb = 1, total = 1;
	int i;
	for (i = 0; i < ndims; i++) { na *= adims[i]; nb *= bdims[i]; }
	for (i = 0; i < ndims - 2; i++) total *= cdims[i];
	/* l-ten/backprop.cpp:491 */
	if (dA) memset(dA, 0, sizeof(float) * na);
	if (dB) memset(dB, 0, sizeof(float) * nb);
	if (total == 0) return 0;
	do {
		const float* top = dC + bcast_offset(idx, cdims, sc, ndims - 2);
		uint64_t oa = bcast_offset(idx, adims, sa, ndims - 2);
		uint64_t ob = bcast_offset(idx, bdims, sb, ndims - 2);
		if (dA) /* :509  dA[M x K] += dC[M x N] * B[K x N]^T */
			oracle_sgemm(0, 1, M, K, N, 1.0f, top, N, B + ob, N, 1.0f, dA + oa, K);
		if (dB) /* :520  dB[K x N] += A[M x K]^T * dC[M x N] */
			oracle_sgemm(1, 0, K, N, M, 1.0f, A + oa, K, top, N, 1.0f, dB + ob, N);
	} while (next_index(idx, cdims, ndims - 2));
	return 0;
}

/* --------------------------------------------------------------------- Conv2d */

void oracle_conv2d_forward(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                           uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                           const float* x, const float* w, float* y, float* col)
{
	uint64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1; /* l-ten/conv2d.cpp:102-103 */
	uint64_t Kc = Cin * kh * kw, HW = Ho * Wo, n;
	for (n = 0; n < N; n++) { /* :136-143 */
		oracle_im2col_f32(x + n * Cin * H * W, Cin, H, W, kh, kw, ph, pw, sh, sw, col);
		oracle_sgemm(0, 0, Cout, HW, Kc, 1.0f, w, Kc, col, HW, 0.0f, y + n * Cout * HW, HW);
	}
}

int oracle_conv2dq_forward(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                           uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                           const uint8_t* x, const uint8_t* w, const int32_t* bias,
                           const oracle_qparams* qp_in_wt_out, uint8_t* y, int32_t* acc_out)
{
	/* l-ten/conv2d.cpp:318-372: per image, u8 im2col (zero bytes outside the image) then
	 * quantized_matmul(false, false, Cout, Ho*Wo, Cin*kh*kw) with qparams[0] = weights,
	 * qparams[1] = input (:347-349).  The bias, when given, is indexed by the GEMM column, i.e. by
	 * output position (l-ten/math_fns.cpp:1470-1473): it must hold Ho*Wo ints. */
	uint64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
	uint64_t Kc = Cin * kh * kw, HW = Ho * Wo, n;
	oracle_qparams qp[3];
	uint8_t* col = (uint8_t*)malloc(Kc * HW + 1);
	int32_t* ws = (int32_t*)malloc(sizeof(int32_t) * (Cout + HW + 1));
	int rc = 0;
	qp[0] = qp_in_wt_out[1];
	qp[1] = qp_in_wt_out[0];
	qp[2] = qp_in_wt_out[2];
	for (n = 0; n < N && rc == 0; n++) {
		oracle_im2col_u8(x + n * Cin * H * W, Cin, H, W, kh, kw, ph, pw, sh, sw, col);
		rc = oracle_quantized_matmul(0, 0, Cout, HW, Kc, 1, w, col, 0, y + n * Cout * HW, qp, bias, ws,
		                             acc_out ? acc_out + n * Cout * HW : NULL);
	}
	free(col);
	free(ws);
	return rc;
}

void oracle_conv2d_wgrad(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                         uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                         const float* x, const float* dy, float* dw, float* col)
{
	uint64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
	uint64_t Kc = Cin * kh * kw, HW = Ho * Wo, n;
	memset(dw, 0, sizeof(float) * Cout * Kc); /* l-ten/backprop.cpp:1943 */
	for (n = 0; n < N; n++) {                /* :1949-1953 */
		oracle_im2col_f32(x + n * Cin * H * W, Cin, H, W, kh, kw, ph, pw, sh, sw, col);
		oracle_sgemm(0, 1, Cout, Kc, HW, 1.0f, dy + n * Cout * HW, HW, col, HW, 1.0f, dw, Kc);
	}
}

void oracle_conv2d_dgrad(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                         uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                         const float* w, const float* dy, float* dx, float* col)
{
	uint64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
	uint64_t Kc = Cin * kh * kw, HW = Ho * Wo, n;
	memset(dx, 0, sizeof(float) * N * Cin * H * W); /* l-ten/backprop.cpp:1957 */
	for (n = 0; n < N; n++) {                      /* :1963-1967 */
		oracle_sgemm(1, 0, Kc, HW, Cout, 1.0f, w, Kc, dy + n * Cout * HW, HW, 0.0f, col, HW);
		oracle_col2im_f32(col, Cin, H, W, kh, kw, ph, pw, sh, sw, dx + n * Cin * H * W);
	}
}

/* --------------------------------------------------------------------- element-wise pieces of the MLP step */

void oracle_relu(const float* src, float* dst, uint64_t n)
{
	uint64_t i; /* l-ten/layers.cpp:32-43 */
	for (i = 0; i < n; i++) dst[i] = src[i] > 0 ? src[i] : 0;
}

void oracle_relu_backward(const float* top, const float* input, float* bottom, uint64_t n)
{
	uint64_t i; /* l-ten/backprop.cpp:2300-2311 */
	for (i = 0; i < n; i++) bottom[i] = input[i] > 0 ? top[i] : 0;
}

void oracle_log_softmax(uint64_t rows, uint64_t cols, const float* x, float* y)
{
	/* l-ten/layers.cpp:93-114 along the last dimension: max, x - max, exp, sum (in index order), exps / sum, log */
	uint64_t r, c;
	for (r = 0; r < rows; r++) {
		const float* xr = x + r * cols;
		float m = xr[0], sum = 0.0f;
		for (c = 1; c < cols; c++) if (xr[c] > m) m = xr[c];
		for (c = 0; c < cols; c++) sum += expf(xr[c] - m);
		for (c = 0; c < cols; c++) y[r * cols + c] = logf(expf(xr[c] - m) / sum);
	}
}

void oracle_log_softmax_backward(uint64_t rows, uint64_t cols, const float* y, const float* dy, float* dx)
{
	/* The chain of l-ten's backward functions for log, div, sum, exp, sub and max collapses to
	 * dx = dy - exp(y) * sum_j dy_j (the two paths through max cancel). */
	uint64_t r, c;
	for (r = 0; r < rows; r++) {
		float s = 0.0f;
		for (c = 0; c < cols; c++) s += dy[r * cols + c];
		for (c = 0; c < cols; c++) dx[r * cols + c] = dy[r * cols + c] - expf(y[r * cols + c]) * s;
	}
}

float oracle_nll_loss(const float* input, const float* target, uint64_t len, uint64_t batch)
{
	uint64_t i; /* l-ten/layers.cpp:243-249 */
	float val = 0;
	for (i = 0; i < len; i++) val += input[i] * target[i];
	return val * (-1.0f / batch);
}

void oracle_nll_backward(const float* target, uint64_t len, uint64_t batch, float top, float* bottom)
{
	uint64_t i; /* l-ten/backprop.cpp:3986-4005: bottom = (-1 / batch * top) * target */
	float scale = -1.0f / (float)batch;
	scale *= top;
	for (i = 0; i < len; i++) bottom[i] = scale * target[i];
}

int oracle_mlp_step(uint64_t batch, int layers, const uint64_t* sizes, const float* X, const float* const* W,
                    const float* const* b, const float* target, float* loss, float* logp, float** dW, float** db,
                    float* dX)
{
	/* FullyConnected (+ bias) with relu between the layers, log_softmax, nll_loss, then backward() from the loss:
	 * the network of l-ten's MNIST tests (tests/nn_tests.cpp) with the sizes of the caller's choice. */
	float* act[17];
	float* pre[17];
	float *g, *g2;
	uint64_t maxw = 0;
	int l, rc = 0;
	if (layers < 1 || layers > 16) return -1;
	for (l = 0; l <= layers; l++) if (sizes[l] > maxw) maxw = sizes[l];
	act[0] = (float*)X;
	for (l = 0; l < layers; l++) {
		pre[l + 1] = (float*)malloc(sizeof(float) * batch * sizes[l + 1]);
		act[l + 1] = (l + 1 < layers) ? (float*)malloc(sizeof(float) * batch * sizes[l + 1]) : pre[l + 1];
		oracle_fc_forward(batch, sizes[l], sizes[l + 1], act[l], W[l], b ? b[l] : NULL, pre[l + 1]);
		if (l + 1 < layers) oracle_relu(pre[l + 1], act[l + 1], batch * sizes[l + 1]);
	}
	oracle_log_softmax(batch, sizes[layers], pre[layers], logp);
	*loss = oracle_nll_loss(logp, target, batch * sizes[layers], batch);

	g = (float*)malloc(sizeof(float) * batch * maxw);
	g2 = (float*)malloc(sizeof(float) * batch * maxw);
	oracle_nll_backward(target, batch * sizes[layers], batch, 1.0f, g2);
	oracle_log_softmax_backward(batch, sizes[layers], logp, g2, g);
	for (l = layers - 1; l >= 0; l--) {
		if (db && db[l]) memset(db[l], 0, sizeof(float) * sizes[l + 1]);
		oracle_fc_backward(batch, sizes[l], sizes[l + 1], act[l], W[l], g, (l > 0 || dX) ? g2 : NULL, dW[l], (b && db) ? db[l] : NULL);
		if (l > 0) oracle_relu_backward(g2, pre[l], g, batch * sizes[l]);
		else if (dX) memcpy(dX, g2, sizeof(float) * batch * sizes[0]);
	}
	for (l = 0; l < layers; l++) {
		if (l + 1 < layers) free(act[l + 1]);
		free(pre[l + 1]);
	}
	free(g);
	free(g2);
	return rc;
}

/* --------------------------------------------------------------------- quantization helpers */

void oracle_min_max(const float* data, uint64_t len, float* min_val, float* max_val)
{
	uint64_t i; /* l-ten/utils.cpp:198-225 */
	float lo = data[0], hi = data[0];
	for (i = 0; i < len; i++) {
		if (data[i] > hi) hi = data[i];
		if (data[i] < lo) lo = data[i];
	}
	*min_val = lo;
	*max_val = hi;
}

void oracle_compute_qparams(float min_val, float max_val, oracle_qparams* qp)
{
	/* l-ten/utils.cpp:265-286 */
	float zero_point;
	min_val = (0.f < min_val) ? 0.f : min_val; /* std::min(min_val, 0.f) */
	max_val = (max_val < 0.f) ? 0.f : max_val; /* std::max(max_val, 0.f) */
	qp->scale = (max_val - min_val) / (255.f - 0.f);
	zero_point = 0.f - min_val / qp->scale;
	qp->zero_point = (uint8_t)roundf(zero_point);
}

void oracle_quantize_u8(const float* data, uint8_t* q, uint64_t len, const oracle_qparams* qp)
{
	uint64_t i; /* l-ten/utils.cpp:241-252 */
	for (i = 0; i < len; i++) {
		float val = (float)qp->zero_point + data[i] / qp->scale;
		val = (val < 255.f) ? val : 255.f; /* std::min(255.f, val) */
		val = (0.f < val) ? val : 0.f;     /* std::max(0.f, val)   */
		q[i] = (uint8_t)roundf(val);
	}
}

void oracle_quantize_i32(const float* data, int32_t* q, uint64_t len, const oracle_qparams* qp)
{
	/* l-ten/utils.cpp:227-239: clamp to [(float)INT_MIN, (float)INT_MAX] (the upper bound rounds up to 2^31), round
	 * half away from zero, convert: what does not fit an int comes out of x86's conversion as 0x80000000 */
	uint64_t i;
	const float lowest = -2147483648.0f, highest = 2147483648.0f;
	for (i = 0; i < len; i++) {
		float val = (float)qp->zero_point + data[i] / qp->scale, r;
		val = (val < highest) ? val : highest;
		val = (lowest < val) ? val : lowest;
		r = roundf(val);
		q[i] = (r >= -2147483648.0f && r < 2147483648.0f) ? (int32_t)r : (int32_t)0x80000000u;
	}
}

void oracle_dequantize_u8(float* data, const uint8_t* q, uint64_t len, const oracle_qparams* qp)
{
	uint64_t i; /* l-ten/utils.cpp:254-262 */
	for (i = 0; i < len; i++) data[i] = qp->scale * (float)((int)q[i] - (int)qp->zero_point);
}

/* --------------------------------------------------------------------- optimizer steps */

void oracle_sgd_step(float* w, float* g, float* v, uint64_t n, float mo, float wd, float lr)
{
	uint64_t j; /* l-ten/optimizer.cpp:52-57; the gradient buffer is overwritten with the decayed gradient */
	for (j = 0; j < n; j++) {
		g[j] = wd * w[j] + g[j];
		v[j] = v[j] * mo + (1.0f - mo) * g[j];
		w[j] = w[j] - (v[j] * lr);
	}
}

void oracle_adam_step(float* w, const float* g, float* v, float* s, uint64_t n, float lr, float beta1, float beta2,
                      uint64_t iteration)
{
	/* l-ten/optimizer.cpp:139-155, the eight element-wise passes applied per element in the same order */
	uint64_t j;
	const float epsilon = 1.0e-8f;
	const float bc1 = 1.0f - powf(beta1, (float)iteration), bc2 = 1.0f - powf(beta2, (float)iteration);
	const float a1 = 1.0f - beta1, a2 = 1.0f - beta2, inv2 = 1.0f / bc2, step = -(1.0f / bc1) * lr;
	for (j = 0; j < n; j++) {
		float scratch;
		v[j] = a1 * g[j] + beta1 * v[j];          /* cpu_axpby */
		scratch = g[j] * g[j];                     /* cpu_mul   */
		s[j] = a2 * scratch + beta2 * s[j];        /* cpu_axpby */
		scratch = inv2 * s[j];                     /* cpu_mul   */
		scratch = powf(scratch, 0.5f);             /* cpu_powx  */
		scratch = epsilon + scratch;               /* cpu_add   */
		scratch = v[j] / scratch;                  /* cpu_div   */
		w[j] = (step == 1.0f) ? w[j] + scratch : w[j] + step * scratch; /* cpu_axpy */
	}
}
