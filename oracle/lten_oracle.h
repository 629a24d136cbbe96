/* TEST INFRASTRUCTURE ONLY — the CPU oracle for the GEMM hot path.
 *
 * A from-scratch restatement, in plain C, of the l-ten CPU algorithms that the HIP
 * path must reproduce.  Only tests, the smoke check and the benchmark's CPU-baseline
 * leg may load this library, and only as the checker; the product library never
 * links, loads or falls back to it.
 *
 * Pinning status (what each function has been checked against, see tests/):
 *   oracle_requantize, oracle_quantized_matmul  pinned: the compiled l-ten CPU path
 *       (dense sweeps + all four transpose modes), the int64 closed form
 *       sum_k (A-zpA)(B-zpB), zero-point invariants, committed golden vectors.
 *   oracle_sgemm / oracle_sgemm_f64            pinned: l-ten's matmul_test and fc_test
 *       vectors, integer-valued exactness, the compiled l-ten cpu_gemm<float>.
 *   oracle_im2col / oracle_col2im              pinned: the compiled l-ten templates
 *       (bit-exact), a direct 7-loop convolution, adjointness <im2col x, c> = <x, col2im c>.
 *   oracle_fc_* / oracle_matmul_* / oracle_conv2d_*  pinned: compiled l-ten layers,
 *       reference-held vectors (fc_test, matmul_test), finite differences.
 *   oracle_conv2dq_forward                     pinned: the compiled l-ten Conv2d_q layer
 *       (golden cases), the int64 closed form with zero bytes as padding, invariants.
 */
#ifndef LTEN_ORACLE_H
#define LTEN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same layout as l-ten's QuantizationParams (l-ten/math_fns.h:12-16). */
typedef struct {
	float   scale;
	uint8_t zero_point;
} oracle_qparams;

/* l-ten/math_fns.cpp:1474 — (unsigned char)((real_multiplier * element) + zero_point):
 * int->float (nearest even), unfused multiply, unfused add, truncate toward zero to
 * int32 with the x86 "integer indefinite" value 0x80000000 for NaN / out of range,
 * then keep the low byte.  No rounding, no saturation. */
uint8_t oracle_requantize(float real_multiplier, int32_t element, uint8_t zero_point);

/* l-ten/math_fns.cpp:1436 — qpA.scale * qpB.scale / qpC.scale, left to right in fp32. */
float oracle_real_multiplier(float scale_a, float scale_b, float scale_c);

/* l-ten/math_fns.cpp:1311-1478 quantized_matmul.  workspace holds N + M ints
 * (row_vector then col_vector, :1325-1326).  When acc_out is not NULL it receives
 * the corrected int32 `element` of :1469-1473 for every output (M*N ints).
 * Returns 0, or -1 for alpha != 1 || beta != 0 (:1331-1334). */
int oracle_quantized_matmul(int transpose_a, int transpose_b, uint64_t M, uint64_t N, uint64_t K,
                            uint8_t alpha, const uint8_t* A, const uint8_t* B, uint8_t beta, uint8_t* C,
                            const oracle_qparams* qparams, const int32_t* bias, int32_t* workspace,
                            int32_t* acc_out);

/* l-ten/math_fns.cpp:771-836 generic_matmul behind cpu_gemm<float> (:1205-1282), with
 * leading dimensions: C = beta*C (overwrite when beta == 0), then C[m][n] +=
 * (alpha*op(A)[m][k]) * op(B)[k][n] accumulated in fp32 in k order. */
void oracle_sgemm(int trans_a, int trans_b, uint64_t M, uint64_t N, uint64_t K, float alpha,
                  const float* A, uint64_t lda, const float* B, uint64_t ldb, float beta,
                  float* C, uint64_t ldc);

/* Same contract, products and sums carried in fp64 and rounded once: the "exact"
 * value that bounds the error of any fp32 summation order. */
void oracle_sgemm_f64(int trans_a, int trans_b, uint64_t M, uint64_t N, uint64_t K, float alpha,
                      const float* A, uint64_t lda, const float* B, uint64_t ldb, float beta,
                      float* C, uint64_t ldc);

/* The same arithmetic as oracle_sgemm, rows spread over `threads` workers in blocks
 * of 4 rows taken round-robin, as l-ten's matmul_mp does (l-ten/math_fns.cpp:1104-1202).
 * Used for CPU-baseline timing when the compiled reference is not available. */
void oracle_sgemm_mt(int trans_a, int trans_b, uint64_t M, uint64_t N, uint64_t K, float alpha,
                     const float* A, uint64_t lda, const float* B, uint64_t ldb, float beta,
                     float* C, uint64_t ldc, int threads);

/* l-ten/im_col.h:5-33 and :35-57 (Caffe semantics; col2im accumulates into im). */
void oracle_im2col_f32(const float* im, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                       uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, float* col);
void oracle_im2col_u8(const uint8_t* im, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                      uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, uint8_t* col);
void oracle_col2im_f32(const float* col, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                       uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, float* im);

/* l-ten/fully_connected.cpp:58-189 (CPU branch :106-125): Y = X W^T (+ ones bias). */
void oracle_fc_forward(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W,
                       const float* bias, float* Y);
/* l-ten/backprop.cpp:2083-2186 (CPU branch): dX = dY W; dW = dY^T X; db += colsum(dY). */
void oracle_fc_backward(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W,
                        const float* dY, float* dX, float* dW, float* db_accum);

/* l-ten/fully_connected.cpp:322-411: leading dims looped (not folded), M = dims[ndims-2]. */
int oracle_fcq_forward(uint64_t batch, uint64_t M, uint64_t in, uint64_t out, const uint8_t* X,
                       const uint8_t* W, const int32_t* bias, const oracle_qparams* qp_in_wt_out,
                       uint8_t* Y);

/* l-ten/md_array.h:959-1017 + :1209-1282: batched NN GEMM over ndims-2 leading dims,
 * size-1 dims broadcast (coordinate clamped).  cdims receives the result dims. */
int oracle_matmul(int ndims, const uint64_t* adims, const uint64_t* bdims, const float* A,
                  const float* B, uint64_t* cdims, float* C);
/* l-ten/backprop.cpp:400-601 (CPU branch): dA += dC B^T, dB += A^T dC per leading index
 * into zero-filled gradients (broadcast operands accumulate). */
int oracle_matmul_backward(int ndims, const uint64_t* adims, const uint64_t* bdims, const float* A,
                           const float* B, const float* dC, float* dA, float* dB);

/* l-ten/conv2d.cpp:55-197 (CPU branch :134-144): per image im2col + NN GEMM. */
/* l-ten/conv2d.cpp:265-387 Conv2d_q::forward: per image u8 im2col + quantized_matmul(false, false)
 * with the weights as the left operand.  bias (or NULL) holds Ho*Wo ints and is added per output
 * position, as the reference's call does.  acc_out (or NULL) receives the int32 values before the
 * requantize.  Pinned: the compiled Conv2d_q layer (golden cases), composition of pinned parts. */
int oracle_conv2dq_forward(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                           uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                           const uint8_t* x, const uint8_t* w, const int32_t* bias,
                           const oracle_qparams* qp_in_wt_out, uint8_t* y, int32_t* acc_out);

void oracle_conv2d_forward(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                           uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                           const float* x, const float* w, float* y, float* col_scratch);
/* l-ten/backprop.cpp:1941-1954: dW = sum_n dY_n col_n^T (NT GEMM, beta = 1 over images). */
void oracle_conv2d_wgrad(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                         uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                         const float* x, const float* dy, float* dw, float* col_scratch);
/* l-ten/backprop.cpp:1955-1968: per image col = W^T dY_n (TN GEMM) then col2im. */
void oracle_conv2d_dgrad(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                         uint64_t kh, uint64_t kw, uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw,
                         const float* w, const float* dy, float* dx, float* col_scratch);

/* Element-wise pieces that sit between the GEMMs of an MLP training step: relu (l-ten/layers.cpp:9-67),
 * relu_backward (l-ten/backprop.cpp:2282-2327), log_softmax along the last dimension (l-ten/layers.cpp:93-114, a
 * composition of max, sub, exp, sum, div, log) and the collapsed form of its backward chain, nll_loss
 * (l-ten/layers.cpp:212-273) and nll_backward (l-ten/backprop.cpp:3975-4040).  Pinned: a whole training step of the
 * compiled l-ten network (golden case) at 1e-5, finite differences of the loss, closed forms. */
void oracle_relu(const float* src, float* dst, uint64_t n);
void oracle_relu_backward(const float* top, const float* input, float* bottom, uint64_t n);
void oracle_log_softmax(uint64_t rows, uint64_t cols, const float* x, float* y);
void oracle_log_softmax_backward(uint64_t rows, uint64_t cols, const float* y, const float* dy, float* dx);
float oracle_nll_loss(const float* input, const float* target, uint64_t len, uint64_t batch);
void oracle_nll_backward(const float* target, uint64_t len, uint64_t batch, float top, float* bottom);
/* One training step of FullyConnected(+bias) -> relu -> ... -> FullyConnected -> log_softmax -> nll_loss and
 * backward(): sizes[0..layers], W[l] is [sizes[l+1] x sizes[l]], target is one-hot [batch x sizes[layers]].
 * Outputs: loss, logp [batch x sizes[layers]], dW[l], db[l] (may be NULL with b), dX (may be NULL). */
int oracle_mlp_step(uint64_t batch, int layers, const uint64_t* sizes, const float* X, const float* const* W,
                    const float* const* b, const float* target, float* loss, float* logp, float** dW, float** db,
                    float* dX);

/* l-ten/utils.cpp:198-286: GetMinMax, ComputeQuantizationParams, Quantize (uint8 and int), Dequantize.
 * Pinned: the compiled l-ten functions on inputs with ties, out-of-range values, infinities and NaN (golden
 * cases, bit-exact), closed forms (round half away from zero, clamp to [0, 255]). */
void oracle_min_max(const float* data, uint64_t len, float* min_val, float* max_val);
void oracle_compute_qparams(float min_val, float max_val, oracle_qparams* qp);
void oracle_quantize_u8(const float* data, uint8_t* q, uint64_t len, const oracle_qparams* qp);
void oracle_quantize_i32(const float* data, int32_t* q, uint64_t len, const oracle_qparams* qp);
void oracle_dequantize_u8(float* data, const uint8_t* q, uint64_t len, const oracle_qparams* qp);

/* SGDOptimizer::step and AdamOptimizer::step for one parameter tensor (l-ten/optimizer.cpp:26-84, 107-186).
 * sgd: g = wd*w + g (stored), v = v*mo + (1-mo)*g, w = w - v*lr.  adam: v, s are the two history buffers,
 * iteration counts from 1.  Pinned: the compiled optimizers over several steps (golden case; sgd bit-exact,
 * adam within 1e-6 because of powf), closed forms. */
void oracle_sgd_step(float* w, float* g, float* v, uint64_t n, float mo, float wd, float lr);
void oracle_adam_step(float* w, const float* g, float* v, float* s, uint64_t n, float lr, float beta1, float beta2,
                      uint64_t iteration);

#ifdef __cplusplus
}
#endif
#endif
