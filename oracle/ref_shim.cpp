// Test infrastructure only.
//
// extern "C" doors into the real l-ten CPU path, compiled together with l-ten's own
// sources (see the Makefile's `ref` target).  The functions below only marshal plain
// buffers into l-ten objects and call l-ten; they hold no arithmetic of their own.
// The resulting library validates the C oracle and serves as the "reference" CPU
// baseline.  The product never links or loads it.
#include <cstdint>
#include <cstring>
#include <cstdlib>
#include <vector>
#include "lten.h"
#include "im_col.h"

extern "C" {

// l-ten/math_fns.cpp:1311 quantized_matmul
int ref_quantized_matmul(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, uint8_t alpha,
                         const uint8_t* A, const uint8_t* B, uint8_t beta, uint8_t* C,
                         const float* scales, const uint8_t* zero_points, const int* bias,
                         int* workspace)
{
	QuantizationParams qp[3];
	for (int i = 0; i < 3; i++) { qp[i].scale = scales[i]; qp[i].zero_point = zero_points[i]; }
	try {
		quantized_matmul(tA != 0, tB != 0, M, N, K, alpha, const_cast<uint8_t*>(A),
		                 const_cast<uint8_t*>(B), beta, C, qp, const_cast<int*>(bias), workspace);
	} catch (...) { return -1; }
	return 0;
}

// l-ten/math_fns.cpp:1258 cpu_gemm<float> (threadpool + AVX fallback build).
// A is copied because matmul_mp scales it in place.  Full 16-column blocks are written with
// aligned 32-byte stores (l-ten/math_fns.cpp:994-1002), so C goes through a 32-byte aligned
// bounce buffer and, once N >= 16 brings that path in, N must keep rows aligned (N % 8 == 0).
int ref_cpu_gemm_f32(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, float alpha,
                     const float* A, const float* B, float beta, float* C)
{
	if (N >= 16 && (N & 7) != 0) return -2;  // would fault inside l-ten; callers pick other shapes
	float* Ac = static_cast<float*>(aligned_alloc(32, ((M * K * 4 + 31) / 32) * 32));
	float* Cc = static_cast<float*>(aligned_alloc(32, ((M * N * 4 + 31) / 32) * 32));
	memcpy(Ac, A, M * K * 4);
	memcpy(Cc, C, M * N * 4);
	int rc = 0;
	try {
		cpu_gemm<float>(tA != 0, tB != 0, M, N, K, alpha, Ac, const_cast<float*>(B), beta, Cc);
	} catch (...) { rc = -1; }
	memcpy(C, Cc, M * N * 4);
	free(Ac);
	free(Cc);
	return rc;
}

// l-ten/im_col.h:5 im2col_cpu, :35 col2im_cpu
void ref_im2col_f32(const float* im, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                    uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, float* col)
{
	im2col_cpu<float>(im, C, H, W, kh, kw, ph, pw, sh, sw, col);
}

void ref_col2im_f32(const float* col, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                    uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, float* im)
{
	col2im_cpu<float>(col, C, H, W, kh, kw, ph, pw, sh, sw, im);
}

void ref_im2col_u8(const uint8_t* im, uint64_t C, uint64_t H, uint64_t W, uint64_t kh, uint64_t kw,
                   uint64_t ph, uint64_t pw, uint64_t sh, uint64_t sw, uint8_t* col)
{
	im2col_cpu<uint8_t>(im, C, H, W, kh, kw, ph, pw, sh, sw, col);
}

// lten::FullyConnected forward (+ backward from a given upstream gradient), l-ten/fully_connected.cpp:58,
// l-ten/backprop.cpp:2083.  x: {1,1,M,in}. Outputs may be null.
int ref_fc_f32(uint64_t M, uint64_t in, uint64_t out, const float* x, const float* w, const float* bias,
               const float* dy, float* y, float* dx, float* dw, float* db)
{
	try {
		lten::Tensor X = lten::TensorFromBuffer({ 1, 1, M, in }, const_cast<float*>(x), false);
		X.set_autograd(true);
		lten::FullyConnected fc(in, out, bias != nullptr);
		fc.init();
		memcpy(fc.get_weights()->get_data_ptr(), w, out * in * 4);
		if (bias) memcpy(fc.get_bias()->get_data_ptr(), bias, out * 4);
		lten::Tensor Y = fc.forward(X);
		if (y) memcpy(y, Y.get_data_ptr(), M * out * 4);
		if (dy) {
			MultiDimArray<float> top;
			top.Allocate({ 1, 1, M, out }, const_cast<float*>(dy), false);
			Y.backward(&top);
			if (dx) memcpy(dx, X.get_grad_ptr(), M * in * 4);
			if (dw) memcpy(dw, fc.get_weights()->get_grad_ptr(), out * in * 4);
			if (db && bias) memcpy(db, fc.get_bias()->get_grad_ptr(), out * 4);
		}
	} catch (...) { return -1; }
	return 0;
}

// l-ten/utils.cpp:198-286 quantization helpers, as compiled.
void ref_min_max(const float* data, uint64_t len, float* lo, float* hi) { GetMinMax(const_cast<float*>(data), len, lo, hi); }
void ref_compute_qparams(float lo, float hi, float* scale, uint8_t* zero_point)
{
	QuantizationParams qp;
	ComputeQuantizationParams(lo, hi, &qp);
	*scale = qp.scale;
	*zero_point = qp.zero_point;
}
void ref_quantize_u8(const float* data, uint8_t* q, uint64_t len, float scale, uint8_t zero_point)
{
	QuantizationParams qp;
	qp.scale = scale; qp.zero_point = zero_point;
	Quantize(const_cast<float*>(data), q, len, &qp);
}
void ref_quantize_i32(const float* data, int* q, uint64_t len, float scale, uint8_t zero_point)
{
	QuantizationParams qp;
	qp.scale = scale; qp.zero_point = zero_point;
	Quantize(const_cast<float*>(data), q, len, &qp);
}
void ref_dequantize_u8(float* data, const uint8_t* q, uint64_t len, float scale, uint8_t zero_point)
{
	QuantizationParams qp;
	qp.scale = scale; qp.zero_point = zero_point;
	Dequantize(data, const_cast<uint8_t*>(q), len, &qp);
}

// SGDOptimizer / AdamOptimizer (l-ten/optimizer.cpp) on a one-layer network whose weight tensor holds `n` values:
// `steps` calls of step(), gradient `g` restored before each (SGD overwrites it).  kind 0 = SGD (p = mo, wd, lr),
// kind 1 = Adam (p = lr, beta1, beta2).
namespace {
struct OneLayerNet : public lten::NeuralNetwork {
	explicit OneLayerNet(uint64_t n) { fc = register_module("fc", lten::FullyConnected(n, 1, false)); }
	lten::FullyConnected* fc;
};
}
int ref_optimizer_steps(int kind, uint64_t n, int steps, const float* p, float* w, const float* g)
{
	try {
		OneLayerNet net(n);
		lten::Tensor* wt = net.fc->get_weights();
		memcpy(wt->get_data_ptr(), w, n * 4);
		lten::Tensor X = lten::AllocateTensor({ 1, 1, 1, n }, nullptr);
		memset(X.get_data_ptr(), 0, n * 4);
		lten::Tensor Y = net.fc->forward(X);
		Y.backward();  // allocates the weight's gradient buffer
		lten::SGDOptimizer sgd;
		lten::AdamOptimizer adam;
		lten::Optimizer* opt;
		if (kind == 0) { sgd.set_momentum(p[0]); sgd.set_weight_decay(p[1]); sgd.set_learning_rate(p[2]); opt = &sgd; }
		else { adam.set_learning_rate(p[0]); adam.set_beta1(p[1]); adam.set_beta2(p[2]); opt = &adam; }
		opt->attach_network(net);
		for (int s = 0; s < steps; s++) {
			memcpy(wt->get_grad_ptr(), g, n * 4);
			opt->step();
		}
		memcpy(w, wt->get_data_ptr(), n * 4);
	} catch (...) { return -1; }
	return 0;
}

// One training step of l-ten's MLP (tests/nn_tests.cpp): FullyConnected(+bias) -> relu -> ... -> FullyConnected ->
// log_softmax(dim 3) -> nll_loss -> backward().  x: {batch,1,1,sizes[0]}, target one-hot {batch,1,1,sizes[layers]}.
int ref_mlp_step(uint64_t batch, int layers, const uint64_t* sizes, const float* x, const float* const* w,
                 const float* const* b, const float* target, float* loss, float* logp, float** dw, float** db, float* dx)
{
	try {
		lten::Tensor X = lten::TensorFromBuffer({ batch, 1, 1, sizes[0] }, const_cast<float*>(x), false);
		X.set_autograd(true);
		lten::Tensor T = lten::TensorFromBuffer({ batch, 1, 1, sizes[layers] }, const_cast<float*>(target), false);
		std::vector<lten::FullyConnected*> fcs;
		for (int l = 0; l < layers; l++) {
			lten::FullyConnected* fc = new lten::FullyConnected(sizes[l], sizes[l + 1], b != nullptr);
			fc->init();
			memcpy(fc->get_weights()->get_data_ptr(), w[l], sizes[l + 1] * sizes[l] * 4);
			if (b) memcpy(fc->get_bias()->get_data_ptr(), b[l], sizes[l + 1] * 4);
			fcs.push_back(fc);
		}
		lten::Tensor h = X;
		for (int l = 0; l < layers; l++) {
			h = fcs[l]->forward(h);
			if (l + 1 < layers) h = lten::relu(h);
		}
		lten::Tensor lp = lten::log_softmax(h, 3);
		lten::Tensor L = lten::nll_loss(lp, T);
		*loss = *static_cast<float*>(L.get_data_ptr());
		memcpy(logp, lp.get_data_ptr(), batch * sizes[layers] * 4);
		L.backward();
		for (int l = 0; l < layers; l++) {
			memcpy(dw[l], fcs[l]->get_weights()->get_grad_ptr(), sizes[l + 1] * sizes[l] * 4);
			if (b && db) memcpy(db[l], fcs[l]->get_bias()->get_grad_ptr(), sizes[l + 1] * 4);
		}
		if (dx) memcpy(dx, X.get_grad_ptr(), batch * sizes[0] * 4);
		for (auto fc : fcs) delete fc;
	} catch (...) { return -1; }
	return 0;
}

// lten::FullyConnected_q forward, l-ten/fully_connected.cpp:322.  x: {batch,M,in} u8.
int ref_fcq_u8(uint64_t batch, uint64_t M, uint64_t in, uint64_t out, const uint8_t* x, const uint8_t* w,
               const int* bias, const float* scales, const uint8_t* zero_points, uint8_t* y)
{
	try {
		lten::TensorOps ops;
		ops.data_type = lten::UINT8;
		lten::Tensor X = lten::TensorFromBuffer({ batch, M, in }, const_cast<uint8_t*>(x), false, &ops);
		lten::FullyConnected_q fc(in, out, bias != nullptr);
		fc.init();
		fc.train(false);
		memcpy(fc.get_weights()->get_data_ptr(), w, out * in);
		if (bias) memcpy(fc.get_bias()->get_data_ptr(), bias, out * 4);
		QuantizationParams qi, qw, qo;
		qi.scale = scales[0]; qi.zero_point = zero_points[0];
		qw.scale = scales[1]; qw.zero_point = zero_points[1];
		qo.scale = scales[2]; qo.zero_point = zero_points[2];
		fc.set_qparams_in(qi);
		fc.set_qparams_params(&qw, 1);
		fc.set_qparams_out(qo);
		lten::Tensor Y = fc.forward(X);
		memcpy(y, Y.get_data_ptr(), batch * M * out);
	} catch (...) { return -1; }
	return 0;
}

// lten::Conv2d_q forward (no bias: l-ten's own call indexes the bias by output position), l-ten/conv2d.cpp:265.
int ref_conv2dq_u8(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph, int pw,
                   int sh, int sw, const uint8_t* x, const uint8_t* w, const float* scales, const uint8_t* zero_points,
                   uint8_t* y)
{
	try {
		lten::TensorOps ops;
		ops.data_type = lten::UINT8;
		lten::Tensor X = lten::TensorFromBuffer({ N, Cin, H, W }, const_cast<uint8_t*>(x), false, &ops);
		lten::Conv2d_q conv((int)Cin, (int)Cout, false, kh, kw, ph, pw, sh, sw);
		conv.init();
		conv.train(false);
		memcpy(conv.get_weights()->get_data_ptr(), w, Cout * Cin * kh * kw);
		QuantizationParams qi, qw, qo;
		qi.scale = scales[0]; qi.zero_point = zero_points[0];
		qw.scale = scales[1]; qw.zero_point = zero_points[1];
		qo.scale = scales[2]; qo.zero_point = zero_points[2];
		conv.set_qparams_in(qi);
		conv.set_qparams_params(&qw, 1);
		conv.set_qparams_out(qo);
		lten::Tensor Y = conv.forward(X);
		uint64_t Ho = (H + 2 * ph - kh) / sh + 1;
		uint64_t Wo = (W + 2 * pw - kw) / sw + 1;
		memcpy(y, Y.get_data_ptr(), N * Cout * Ho * Wo);
	} catch (...) { return -1; }
	return 0;
}

// lten::Conv2d forward + weight/data gradient, l-ten/conv2d.cpp:55, l-ten/backprop.cpp:1841.
int ref_conv2d_f32(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph, int pw,
                   int sh, int sw, const float* x, const float* w, const float* dy, float* y, float* dw, float* dx)
{
	try {
		lten::Tensor X = lten::TensorFromBuffer({ N, Cin, H, W }, const_cast<float*>(x), false);
		X.set_autograd(true);
		lten::Conv2d conv((int)Cin, (int)Cout, false, kh, kw, ph, pw, sh, sw);
		conv.init();
		memcpy(conv.get_weights()->get_data_ptr(), w, Cout * Cin * kh * kw * 4);
		lten::Tensor Y = conv.forward(X);
		uint64_t Ho = (H + 2 * ph - kh) / sh + 1;
		uint64_t Wo = (W + 2 * pw - kw) / sw + 1;
		if (y) memcpy(y, Y.get_data_ptr(), N * Cout * Ho * Wo * 4);
		if (dy) {
			MultiDimArray<float> top;
			top.Allocate({ N, Cout, Ho, Wo }, const_cast<float*>(dy), false);
			Y.backward(&top);
			if (dw) memcpy(dw, conv.get_weights()->get_grad_ptr(), Cout * Cin * kh * kw * 4);
			if (dx) memcpy(dx, X.get_grad_ptr(), N * Cin * H * W * 4);
		}
	} catch (...) { return -1; }
	return 0;
}

// lten::Tensor::matmul (+ backward), l-ten/tensor.h:83, l-ten/md_array.h:959, l-ten/backprop.cpp:400.
// Both operands have `ndims` dims (>= 3 here); leading dims broadcast when 1.
int ref_matmul_f32(int ndims, const uint64_t* adims, const uint64_t* bdims, const float* a, const float* b,
                   const float* dc, float* c, float* da, float* db)
{
	try {
		lten::Tensor A = lten::TensorFromBuffer(adims, ndims, const_cast<float*>(a), false);
		lten::Tensor B = lten::TensorFromBuffer(bdims, ndims, const_cast<float*>(b), false);
		A.set_autograd(true);
		B.set_autograd(true);
		lten::Tensor C = A.matmul(B);
		if (c) memcpy(c, C.get_data_ptr(), C.get_numels() * 4);
		if (dc) {
			MultiDimArray<float> top;
			top.Allocate(C.get_sizes(), ndims, const_cast<float*>(dc), false);
			C.backward(&top);
			if (da) memcpy(da, A.get_grad_ptr(), A.get_numels() * 4);
			if (db) memcpy(db, B.get_grad_ptr(), B.get_numels() * 4);
		}
	} catch (...) { return -1; }
	return 0;
}

int ref_hardware_threads(void)
{
	return (int)std::thread::hardware_concurrency();
}

}  // extern "C"
