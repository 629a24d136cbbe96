// Tests of the host-side layer API on the GPU, written the way l-ten's own unit tests are
// (tests/unit_tests.cpp): tiny hard-coded tensors, forward values and gradients compared with Compare().
// matmul_test and fc_test use l-ten's own inputs and expected vectors; the others check the layer
// plumbing (leading dims, bias, chains of layers, error behaviour) against plain loops.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "lten_gpu.h"
#include "../../include/lten_hip.h"

template <typename Dtype>
static int Compare(const Dtype* A, const Dtype* B, uint64_t len, double error = 0)
{
	for (uint64_t i = 0; i < len; i++)
		if (std::fabs((double)A[i] - (double)B[i]) > error) return -1;
	return 0;
}

static std::vector<float> grad_to_host(lten::Tensor& t)
{
	std::vector<float> out(t.get_numels());
	lten::Tensor cpu = t.to(lten::CPU);
	memcpy(out.data(), cpu.get_grad_ptr(), out.size() * sizeof(float));
	return out;
}

// l-ten tests/unit_tests.cpp:700-764 (run_on_gpu = true); the scalar pick z[1][0][3][1] is passed as a one-hot top gradient
static int matmul_test()
{
	float x_vals[] = { 2, 3, 4, 2, 6, 8, 5, 7, 5, 2, 1, 9, 0, 3, 6, 4, 8, 2, 3, 2, 2, 4, 5, 6 };
	float w_vals[] = { 5, 3, 2, 5, 2, 2, 7, 4, 1, 3, 3, 1 };
	lten::Tensor x = lten::TensorFromBuffer({ 2, 1, 4, 3 }, x_vals, false);
	lten::Tensor w = lten::TensorFromBuffer({ 1, 1, 3, 4 }, w_vals, false);
	x.set_autograd(true);
	w.set_autograd(true);
	x = x.to(lten::GPU);
	w = w.to(lten::GPU);
	lten::Tensor z = x.matmul(w);
	float top_vals[32] = { 0 };
	top_vals[(1 * 4 + 3) * 4 + 1] = 1.0f;
	lten::Tensor top = lten::TensorFromBuffer({ 2, 1, 4, 4 }, top_vals, false).to(lten::GPU);
	z.backward(&top);
	lten::Tensor zc = z.to(lten::CPU);
	float z_vals[] = { 20, 24, 37, 26, 30, 42, 70, 42, 44, 44, 74, 58, 21, 35, 38, 23, 12, 24, 39, 18, 38, 34, 70, 54, 21, 19, 26, 25, 36, 40, 61, 46 };
	float w_grad_vals[] = { 0, 4, 0, 0, 0, 5, 0, 0, 0, 6, 0, 0 };
	float x_grad_vals[] = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 3, 2, 3 };
	if (((float*)zc.get_data_ptr())[(1 * 4 + 3) * 4 + 1] != 40) return -1;
	if (Compare((float*)zc.get_data_ptr(), z_vals, zc.get_numels())) return -1;
	if (Compare(grad_to_host(x).data(), x_grad_vals, 24)) return -1;
	if (Compare(grad_to_host(w).data(), w_grad_vals, 12)) return -1;
	return 0;
}

// l-ten tests/unit_tests.cpp:1231-1331 (run_on_gpu = true)
static int fc_test()
{
	float error = 0.001f;
	float test_wts[] = { 0.0900306f, 0.2447285f, 0.6652409f, 0.0021785f, 0.1189432f, 0.8788782f, 0.1065070f, 0.7869860f, 0.1065070f, 0.0009107f, 0.0003350f, 0.9987543f, 0.0023556f, 0.0473142f, 0.9503303f, 0.0179425f, 0.9796292f, 0.0024283f, 0.5761169f, 0.2119416f, 0.2119416f, 0.0900306f, 0.2447285f, 0.6652409f };
	float x_vals[] = { 2, 3, 4, 2, 6, 8, 5, 7, 5, 2, 1, 9, 0, 3, 6, 4, 8, 2, 3, 2, 2, 4, 5, 6 };
	lten::Tensor x = lten::TensorFromBuffer({ 2, 1, 4, 3 }, x_vals);
	x.set_autograd(true);
	x = x.to(lten::GPU);
	lten::FullyConnected fc(3, 8);
	fc.init();
	for (uint64_t i = 0; i < fc.get_weights()->get_numels(); i++) ((float*)(fc.get_weights()->get_data_ptr()))[i] = test_wts[i];
	fc.to(lten::GPU);
	lten::Tensor z = fc.forward(x);
	float top_vals[64] = { 0 };
	top_vals[(1 * 4 + 3) * 8 + 4] = 1.0f;
	lten::Tensor top = lten::TensorFromBuffer({ 2, 1, 4, 8 }, top_vals, false).to(lten::GPU);
	z.backward(&top);
	lten::Tensor zc = z.to(lten::CPU);
	float z_vals[] = { 3.57521f, 3.8767f, 3.0f, 3.99784f, 3.94798f, 2.98449f, 2.63583f, 3.57521f, 6.97036f, 7.74904f, 5.78699f, 7.99387f, 7.89124f, 5.93309f, 4.11942f, 6.97036f, 5.48946f, 5.23789f, 6.57397f, 5.00067f, 5.09463f, 6.95926f, 5.42388f, 5.48946f, 6.41196f, 8.0332f, 1.95856f, 8.99094f, 8.605f, 1.03737f, 3.27165f, 6.41196f, 4.72563f, 5.6301f, 3.0f, 5.99353f, 5.84392f, 2.95346f, 1.90747f, 4.72563f, 3.64843f, 2.71802f, 6.93493f, 2.00383f, 2.2886f, 7.91366f, 4.42388f, 3.64843f, 2.09003f, 2.00218f, 2.10651f, 2.00091f, 2.00236f, 2.01794f, 2.57612f, 2.09003f, 5.57521f, 5.8767f, 5.0f, 5.99784f, 5.94798f, 4.98449f, 4.63583f, 5.57521f };
	float x_grad_vals[] = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0.0023556f, 0.0473142f, 0.95033f };
	float wt_grad_vals[] = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 4.0f, 5.0f, 6.0f, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
	if (std::fabs(((float*)zc.get_data_ptr())[(1 * 4 + 3) * 8 + 4] - 5.94797564f) > error) return -1;
	if (Compare((float*)zc.get_data_ptr(), z_vals, zc.get_numels(), error)) return -1;
	if (Compare(grad_to_host(x).data(), x_grad_vals, 24, error)) return -1;
	if (Compare(grad_to_host(*fc.get_weights()).data(), wt_grad_vals, 24, error)) return -1;
	return 0;
}

// two FullyConnected layers with bias chained: gradients must flow through the intermediate tensor
static int fc_chain_test()
{
	const uint64_t M = 6, F0 = 5, F1 = 7, F2 = 3;
	std::vector<float> x(M * F0), w1(F1 * F0), b1(F1), w2(F2 * F1), b2(F2), top(M * F2);
	unsigned s = 12345;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (float)((s >> 16) & 0xFF) / 64.0f - 2.0f; };
	for (auto* v : { &x, &w1, &b1, &w2, &b2, &top }) for (auto& e : *v) e = rnd();
	lten::Tensor X = lten::TensorFromBuffer({ 1, M, F0 }, x.data());
	X.set_autograd(true);
	X = X.to(lten::GPU);
	lten::FullyConnected fc1(F0, F1, true), fc2(F1, F2, true);
	fc1.init();
	fc2.init();
	memcpy(fc1.get_weights()->get_data_ptr(), w1.data(), w1.size() * 4);
	memcpy(fc1.get_bias()->get_data_ptr(), b1.data(), b1.size() * 4);
	memcpy(fc2.get_weights()->get_data_ptr(), w2.data(), w2.size() * 4);
	memcpy(fc2.get_bias()->get_data_ptr(), b2.data(), b2.size() * 4);
	fc1.to(lten::GPU);
	fc2.to(lten::GPU);
	lten::Tensor h = fc1.forward(X);
	lten::Tensor y = fc2.forward(h);
	lten::Tensor T = lten::TensorFromBuffer({ 1, M, F2 }, top.data()).to(lten::GPU);
	y.backward(&T);
	// plain loops
	std::vector<float> H(M * F1), Y(M * F2), dH(M * F1, 0), dX(M * F0, 0), dW1(F1 * F0, 0), dW2(F2 * F1, 0), dB1(F1, 0), dB2(F2, 0);
	for (uint64_t m = 0; m < M; m++) for (uint64_t j = 0; j < F1; j++) { float a = b1[j]; for (uint64_t k = 0; k < F0; k++) a += x[m * F0 + k] * w1[j * F0 + k]; H[m * F1 + j] = a; }
	for (uint64_t m = 0; m < M; m++) for (uint64_t j = 0; j < F2; j++) { float a = b2[j]; for (uint64_t k = 0; k < F1; k++) a += H[m * F1 + k] * w2[j * F1 + k]; Y[m * F2 + j] = a; }
	for (uint64_t m = 0; m < M; m++) for (uint64_t j = 0; j < F2; j++) { dB2[j] += top[m * F2 + j]; for (uint64_t k = 0; k < F1; k++) { dH[m * F1 + k] += top[m * F2 + j] * w2[j * F1 + k]; dW2[j * F1 + k] += top[m * F2 + j] * H[m * F1 + k]; } }
	for (uint64_t m = 0; m < M; m++) for (uint64_t j = 0; j < F1; j++) { dB1[j] += dH[m * F1 + j]; for (uint64_t k = 0; k < F0; k++) { dX[m * F0 + k] += dH[m * F1 + j] * w1[j * F0 + k]; dW1[j * F0 + k] += dH[m * F1 + j] * x[m * F0 + k]; } }
	lten::Tensor yc = y.to(lten::CPU);
	const double tol = 1e-3;
	if (Compare((float*)yc.get_data_ptr(), Y.data(), Y.size(), tol)) return -1;
	if (Compare(grad_to_host(X).data(), dX.data(), dX.size(), tol)) return -2;
	if (Compare(grad_to_host(*fc1.get_weights()).data(), dW1.data(), dW1.size(), tol)) return -3;
	if (Compare(grad_to_host(*fc2.get_weights()).data(), dW2.data(), dW2.size(), tol)) return -4;
	if (Compare(grad_to_host(*fc1.get_bias()).data(), dB1.data(), dB1.size(), tol)) return -5;
	if (Compare(grad_to_host(*fc2.get_bias()).data(), dB2.data(), dB2.size(), tol)) return -6;
	return 0;
}

// A whole training step through the layer API, as l-ten's MNIST tests write it: FullyConnected -> relu -> FullyConnected ->
// log_softmax -> nll_loss, then loss.backward(); against plain loops in double precision.
static int mlp_step_test()
{
	const uint64_t B = 5, F0 = 7, F1 = 6, F2 = 4;
	std::vector<float> x(B * F0), w1(F1 * F0), b1(F1), w2(F2 * F1), b2(F2), t(B * F2, 0.0f);
	unsigned s = 777;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (float)((s >> 16) & 0xFF) / 128.0f - 1.0f; };
	for (auto* v : { &x, &w1, &b1, &w2, &b2 }) for (auto& e : *v) e = rnd();
	for (uint64_t m = 0; m < B; m++) t[m * F2 + (m * 3) % F2] = 1.0f;
	lten::Tensor X = lten::TensorFromBuffer({ B, 1, 1, F0 }, x.data());
	X.set_autograd(true);
	X = X.to(lten::GPU);
	lten::Tensor T = lten::TensorFromBuffer({ B, 1, 1, F2 }, t.data()).to(lten::GPU);
	lten::FullyConnected fc1(F0, F1, true), fc2(F1, F2, true);
	fc1.init();
	fc2.init();
	memcpy(fc1.get_weights()->get_data_ptr(), w1.data(), w1.size() * 4);
	memcpy(fc1.get_bias()->get_data_ptr(), b1.data(), b1.size() * 4);
	memcpy(fc2.get_weights()->get_data_ptr(), w2.data(), w2.size() * 4);
	memcpy(fc2.get_bias()->get_data_ptr(), b2.data(), b2.size() * 4);
	fc1.to(lten::GPU);
	fc2.to(lten::GPU);
	lten::Tensor h = fc1.forward(X);
	lten::Tensor a = lten::relu(h);
	lten::Tensor y = fc2.forward(a);
	lten::Tensor lp = lten::log_softmax(y, 3);
	lten::Tensor loss = lten::nll_loss(lp, T);
	loss.backward();
	// plain loops
	std::vector<double> H(B * F1), A(B * F1), Y(B * F2), LP(B * F2), dY(B * F2), dA(B * F1, 0), dH(B * F1), dX(B * F0, 0), dW1(F1 * F0, 0), dW2(F2 * F1, 0), dB1(F1, 0), dB2(F2, 0);
	double L = 0;
	for (uint64_t m = 0; m < B; m++) {
		for (uint64_t j = 0; j < F1; j++) { double v = b1[j]; for (uint64_t k = 0; k < F0; k++) v += (double)x[m * F0 + k] * w1[j * F0 + k]; H[m * F1 + j] = v; A[m * F1 + j] = v > 0 ? v : 0; }
		double mx = -1e300, se = 0;
		for (uint64_t j = 0; j < F2; j++) { double v = b2[j]; for (uint64_t k = 0; k < F1; k++) v += A[m * F1 + k] * w2[j * F1 + k]; Y[m * F2 + j] = v; if (v > mx) mx = v; }
		for (uint64_t j = 0; j < F2; j++) se += exp(Y[m * F2 + j] - mx);
		for (uint64_t j = 0; j < F2; j++) { LP[m * F2 + j] = Y[m * F2 + j] - mx - log(se); L -= LP[m * F2 + j] * t[m * F2 + j] / B; }
		for (uint64_t j = 0; j < F2; j++) dY[m * F2 + j] = (exp(LP[m * F2 + j]) - t[m * F2 + j]) / B;  // softmax - onehot, over the batch
		for (uint64_t j = 0; j < F2; j++) { dB2[j] += dY[m * F2 + j]; for (uint64_t k = 0; k < F1; k++) { dA[m * F1 + k] += dY[m * F2 + j] * w2[j * F1 + k]; dW2[j * F1 + k] += dY[m * F2 + j] * A[m * F1 + k]; } }
		for (uint64_t j = 0; j < F1; j++) { dH[m * F1 + j] = H[m * F1 + j] > 0 ? dA[m * F1 + j] : 0; dB1[j] += dH[m * F1 + j]; for (uint64_t k = 0; k < F0; k++) { dX[m * F0 + k] += dH[m * F1 + j] * w1[j * F0 + k]; dW1[j * F0 + k] += dH[m * F1 + j] * x[m * F0 + k]; } }
	}
	auto f32 = [](const std::vector<double>& v) { return std::vector<float>(v.begin(), v.end()); };
	const double tol = 1e-4;
	lten::Tensor lc = loss.to(lten::CPU);
	float Lf = (float)L;
	if (Compare((float*)lc.get_data_ptr(), &Lf, 1, tol)) return -1;
	lten::Tensor lpc = lp.to(lten::CPU);
	if (Compare((float*)lpc.get_data_ptr(), f32(LP).data(), LP.size(), tol)) return -2;
	if (Compare(grad_to_host(X).data(), f32(dX).data(), dX.size(), tol)) return -3;
	if (Compare(grad_to_host(*fc1.get_weights()).data(), f32(dW1).data(), dW1.size(), tol)) return -4;
	if (Compare(grad_to_host(*fc2.get_weights()).data(), f32(dW2).data(), dW2.size(), tol)) return -5;
	if (Compare(grad_to_host(*fc1.get_bias()).data(), f32(dB1).data(), dB1.size(), tol)) return -6;
	if (Compare(grad_to_host(*fc2.get_bias()).data(), f32(dB2).data(), dB2.size(), tol)) return -7;
	return 0;
}

// A network class in l-ten's style (modules registered in the constructor, l-ten tests/nn_tests.cpp:17-42) trained on the
// device with each optimizer: a 4-class problem whose label is the largest of four fixed projections of the input.
// The loss must fall well below its start value; attach-then-move and move-then-attach must both work.
static int training_test()
{
	class Net : public lten::NeuralNetwork {
	public:
		Net()
		{
			fc1 = register_module("fc1", lten::FullyConnected(8, 32, true));
			fc2 = register_module("fc2", lten::FullyConnected(32, 4, true));
		}
		lten::Tensor forward(lten::Tensor input)
		{
			lten::Tensor h = fc1->forward(input);
			lten::Tensor a = lten::relu(h);
			return fc2->forward(a);
		}
		lten::FullyConnected *fc1, *fc2;
	};
	const uint64_t B = 64, F = 8, C = 4;
	unsigned s = 4242;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (float)((s >> 8) & 0xFFFF) / 32768.0f - 1.0f; };
	std::vector<float> proj(C * F);
	for (auto& e : proj) e = rnd();
	for (int which = 0; which < 2; which++) {
		Net net;
		lten::SGDOptimizer sgd;
		lten::AdamOptimizer adam;
		lten::Optimizer* opt = which == 0 ? (lten::Optimizer*)&sgd : (lten::Optimizer*)&adam;
		sgd.set_learning_rate(0.2f);
		sgd.set_weight_decay(0.0f);
		adam.set_learning_rate(0.01f);
		if (which == 0) { opt->attach_network(net); net.to(lten::GPU); }  // state allocated on the host, moved with the network
		else { net.to(lten::GPU); opt->attach_network(net); }             // state allocated on the device
		float first = 0.0f, last = 0.0f;
		for (int it = 0; it < 300; it++) {
			std::vector<float> x(B * F), t(B * C, 0.0f);
			for (uint64_t m = 0; m < B; m++) {
				for (uint64_t k = 0; k < F; k++) x[m * F + k] = rnd();
				uint64_t best = 0;
				float bv = -1e30f;
				for (uint64_t c = 0; c < C; c++) {
					float v = 0.0f;
					for (uint64_t k = 0; k < F; k++) v += proj[c * F + k] * x[m * F + k];
					if (v > bv) { bv = v; best = c; }
				}
				t[m * C + best] = 1.0f;
			}
			lten::Tensor X = lten::TensorFromBuffer({ B, 1, 1, F }, x.data()).to(lten::GPU);
			lten::Tensor T = lten::TensorFromBuffer({ B, 1, 1, C }, t.data()).to(lten::GPU);
			lten::Tensor y = net.forward(X);
			lten::Tensor lp = lten::log_softmax(y, 3);
			lten::Tensor loss = lten::nll_loss(lp, T);
			loss.backward();
			opt->step();
			opt->zero_grad();
			if (it == 0 || it == 299) {
				lten::Tensor lc = loss.to(lten::CPU);
				(it == 0 ? first : last) = *(float*)lc.get_data_ptr();
			}
		}
		printf("  %s: loss %.4f -> %.4f\n", which == 0 ? "SGD" : "Adam", first, last);
		if (!(last < 0.5f * first) || !(last < 0.7f)) return -1 - which;
	}
	return 0;
}

// Conv2d (with bias) -> relu -> reshape -> FullyConnected trained on the device in l-ten's style: 12 x 12 images with
// a bright 4 x 4 blob in one of four quadrants, the label is the quadrant.
static int conv_training_test()
{
	class Net : public lten::NeuralNetwork {
	public:
		Net()
		{
			conv1 = register_module("conv1", lten::Conv2d(1, 8, true, 3, 3, 1, 1));
			fc1 = register_module("fc1", lten::FullyConnected(8 * 12 * 12, 4, true));
		}
		lten::Tensor forward(lten::Tensor input)
		{
			lten::Tensor c = conv1->forward(input);
			lten::Tensor a = lten::relu(c);
			lten::Tensor flat = a.reshape({ input.get_sizes()[0], 1, 1, 8 * 12 * 12 });
			return fc1->forward(flat);
		}
		lten::Conv2d* conv1;
		lten::FullyConnected* fc1;
	};
	const uint64_t B = 32, S = 12, C = 4;
	unsigned s = 99;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (float)((s >> 8) & 0xFFFF) / 65536.0f; };
	Net net;
	lten::AdamOptimizer adam;
	adam.set_learning_rate(0.003f);
	net.to(lten::GPU);
	adam.attach_network(net);
	float first = 0.0f, last = 0.0f;
	for (int it = 0; it < 150; it++) {
		std::vector<float> x(B * S * S), t(B * C, 0.0f);
		for (uint64_t m = 0; m < B; m++) {
			const int quadrant = (int)(rnd() * 4) & 3, oy = (quadrant / 2) * 6 + 1, ox = (quadrant % 2) * 6 + 1;
			for (uint64_t p = 0; p < S * S; p++) x[m * S * S + p] = 0.2f * rnd();
			for (int dy = 0; dy < 4; dy++) for (int dx = 0; dx < 4; dx++) x[m * S * S + (oy + dy) * S + ox + dx] += 1.0f;
			t[m * C + quadrant] = 1.0f;
		}
		lten::Tensor X = lten::TensorFromBuffer({ B, 1, S, S }, x.data()).to(lten::GPU);
		lten::Tensor T = lten::TensorFromBuffer({ B, 1, 1, C }, t.data()).to(lten::GPU);
		lten::Tensor y = net.forward(X);
		lten::Tensor lp = lten::log_softmax(y, 3);
		lten::Tensor loss = lten::nll_loss(lp, T);
		loss.backward();
		adam.step();
		adam.zero_grad();
		if (it == 0 || it == 149) {
			lten::Tensor lc = loss.to(lten::CPU);
			(it == 0 ? first : last) = *(float*)lc.get_data_ptr();
		}
	}
	printf("  conv net: loss %.4f -> %.4f\n", first, last);
	return (last < 0.2f * first && last < 0.3f) ? 0 : -1;
}

// FullyConnected_q on {2, 3, 37} with bias: every leading index is its own quantized_matmul in l-ten
static int fcq_test()
{
	const uint64_t B = 2, M = 3, K = 37, N = 5;
	std::vector<uint8_t> x(B * M * K), w(N * K);
	std::vector<int> bias(N);
	unsigned s = 99;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (s >> 16) & 0xFF; };
	for (auto& e : x) e = (uint8_t)rnd();
	for (auto& e : w) e = (uint8_t)rnd();
	for (auto& e : bias) e = (int)rnd() * 40 - 5000;
	lten::TensorOps ops;
	ops.data_type = lten::UINT8;
	lten::Tensor X = lten::TensorFromBuffer({ B, M, K }, x.data(), false, &ops).to(lten::GPU);
	lten::FullyConnected_q fc(K, N, true);
	fc.init();
	fc.train(false);
	memcpy(fc.get_weights()->get_data_ptr(), w.data(), w.size());
	memcpy(fc.get_bias()->get_data_ptr(), bias.data(), bias.size() * 4);
	QuantizationParams qi{ 0.02f, 7 }, qw{ 0.013f, 131 }, qo{ 0.7f, 100 };
	fc.set_qparams_in(qi);
	fc.set_qparams_params(&qw, 1);
	fc.set_qparams_out(qo);
	fc.to(lten::GPU);
	lten::Tensor Y = fc.forward(X).to(lten::CPU);
	const float mult = qi.scale * qw.scale / qo.scale;
	std::vector<uint8_t> want(B * M * N);
	for (uint64_t r = 0; r < B * M; r++)
		for (uint64_t n = 0; n < N; n++) {
			int acc = bias[n];
			for (uint64_t k = 0; k < K; k++) acc += ((int)x[r * K + k] - qi.zero_point) * ((int)w[n * K + k] - qw.zero_point);
			volatile float p = mult * (float)acc;
			volatile float sum = p + (float)qo.zero_point;
			want[r * N + n] = (uint8_t)((int)sum & 0xFF);
		}
	return Compare((uint8_t*)Y.get_data_ptr(), want.data(), want.size());
}

// A layer whose weights are written again while it sits on the GPU (what l-ten's load_checkpoint does through
// get_all_weights, l-ten/net.h:227-236): the forward that follows must run on the new weights, not on the int8 copy
// and row sums made for the old ones.  Shape on the direct-to-LDS tiles, zero points that need every correction term.
static int fcq_reload_test()
{
	const uint64_t M = 160, K = 512, N = 256;
	std::vector<uint8_t> x(M * K), w0(N * K), w1(N * K);
	unsigned s = 4321;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (s >> 16) & 0xFF; };
	for (auto& e : x) e = (uint8_t)rnd();
	for (auto& e : w0) e = (uint8_t)rnd();
	for (auto& e : w1) e = (uint8_t)rnd();
	lten::TensorOps ops;
	ops.data_type = lten::UINT8;
	lten::Tensor X = lten::TensorFromBuffer({ 1, M, K }, x.data(), false, &ops).to(lten::GPU);
	lten::FullyConnected_q fc(K, N, false);
	fc.init();
	fc.train(false);
	memcpy(fc.get_weights()->get_data_ptr(), w0.data(), w0.size());
	QuantizationParams qi{ 0.02f, 17 }, qw{ 0.013f, 250 }, qo{ 3.1f, 100 };
	fc.set_qparams_in(qi);
	fc.set_qparams_params(&qw, 1);
	fc.set_qparams_out(qo);
	fc.to(lten::GPU);
	const float mult = qi.scale * qw.scale / qo.scale;
	auto expect = [&](const std::vector<uint8_t>& w, std::vector<uint8_t>& want) {
		want.resize(M * N);
		for (uint64_t r = 0; r < M; r++)
			for (uint64_t n = 0; n < N; n++) {
				int acc = 0;
				for (uint64_t k = 0; k < K; k++) acc += ((int)x[r * K + k] - qi.zero_point) * ((int)w[n * K + k] - qw.zero_point);
				volatile float p = mult * (float)acc;
				volatile float sum = p + (float)qo.zero_point;
				want[r * N + n] = (uint8_t)((int)sum & 0xFF);
			}
	};
	std::vector<uint8_t> want;
	lten::Tensor Y = fc.forward(X).to(lten::CPU);
	expect(w0, want);
	if (Compare((uint8_t*)Y.get_data_ptr(), want.data(), want.size())) return -1;
	// new weights straight into the GPU-resident tensor, as a checkpoint loader does
	std::vector<lten::Tensor*> params = fc.get_all_weights();
	if (lten_hip_copy_to_gpu(params[0]->get_data_ptr(), w1.data(), w1.size()) != 0) return -1;
	Y = fc.forward(X).to(lten::CPU);
	expect(w1, want);
	return Compare((uint8_t*)Y.get_data_ptr(), want.data(), want.size());
}

// Conv2d_q (the 1 -> 10 channel 5x5 layer of l-ten's quantized MNIST network, plus a padded strided one) against plain loops
static int convq_test()
{
	struct Geo { int N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw; } geos[] = { { 3, 1, 28, 28, 10, 5, 5, 0, 0, 1, 1 }, { 2, 12, 9, 11, 6, 3, 3, 1, 2, 2, 1 } };
	unsigned s = 1234;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (s >> 16) & 0xFF; };
	for (const Geo& g : geos) {
		const int Ho = (g.H + 2 * g.ph - g.kh) / g.sh + 1, Wo = (g.W + 2 * g.pw - g.kw) / g.sw + 1, K = g.Cin * g.kh * g.kw;
		std::vector<uint8_t> x((size_t)g.N * g.Cin * g.H * g.W), w((size_t)g.Cout * K);
		for (auto& e : x) e = (uint8_t)rnd();
		for (auto& e : w) e = (uint8_t)rnd();
		lten::TensorOps ops;
		ops.data_type = lten::UINT8;
		lten::Tensor X = lten::TensorFromBuffer({ (uint64_t)g.N, (uint64_t)g.Cin, (uint64_t)g.H, (uint64_t)g.W }, x.data(), false, &ops).to(lten::GPU);
		lten::Conv2d_q conv(g.Cin, g.Cout, false, g.kh, g.kw, g.ph, g.pw, g.sh, g.sw);
		conv.init();
		conv.train(false);
		memcpy(conv.get_weights()->get_data_ptr(), w.data(), w.size());
		QuantizationParams qi{ 0.02f, 9 }, qw{ 0.011f, 120 }, qo{ 0.8f, 90 };
		conv.set_qparams_in(qi);
		conv.set_qparams_params(&qw, 1);
		conv.set_qparams_out(qo);
		conv.to(lten::GPU);
		lten::Tensor Y = conv.forward(X).to(lten::CPU);
		const float mult = qw.scale * qi.scale / qo.scale;  // qparams[0] = weights in l-ten's call
		std::vector<uint8_t> want((size_t)g.N * g.Cout * Ho * Wo);
		for (int n = 0; n < g.N; n++)
			for (int co = 0; co < g.Cout; co++)
				for (int ho = 0; ho < Ho; ho++)
					for (int wo = 0; wo < Wo; wo++) {
						int acc = 0;
						for (int ci = 0; ci < g.Cin; ci++)
							for (int i = 0; i < g.kh; i++)
								for (int j = 0; j < g.kw; j++) {
									const int yy = ho * g.sh - g.ph + i, xx = wo * g.sw - g.pw + j;
									const int xv = (yy >= 0 && yy < g.H && xx >= 0 && xx < g.W) ? x[((size_t)(n * g.Cin + ci) * g.H + yy) * g.W + xx] : 0;
									acc += ((int)w[(size_t)co * K + (ci * g.kh + i) * g.kw + j] - qw.zero_point) * (xv - qi.zero_point);
								}
						volatile float p = mult * (float)acc;
						volatile float sum = p + (float)qo.zero_point;
						want[((size_t)(n * g.Cout + co) * Ho + ho) * Wo + wo] = (uint8_t)((int)sum & 0xFF);
					}
		if (Compare((uint8_t*)Y.get_data_ptr(), want.data(), want.size())) return -1;
	}
	return 0;
}

// Conv2d forward, weight gradient and data gradient against plain loops (stride 2, pad 1, non-square)
static int conv_test()
{
	const int N = 2, Cin = 3, H = 7, W = 9, Cout = 4, kh = 3, kw = 2, ph = 1, pw = 1, sh = 2, sw = 1;
	const int Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
	std::vector<float> x(N * Cin * H * W), w(Cout * Cin * kh * kw), dy(N * Cout * Ho * Wo);
	unsigned s = 7;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (float)((s >> 16) & 0xFF) / 128.0f - 1.0f; };
	for (auto* v : { &x, &w, &dy }) for (auto& e : *v) e = rnd();
	lten::Tensor X = lten::TensorFromBuffer({ (uint64_t)N, (uint64_t)Cin, (uint64_t)H, (uint64_t)W }, x.data());
	X.set_autograd(true);
	X = X.to(lten::GPU);
	lten::Conv2d conv(Cin, Cout, true, kh, kw, ph, pw, sh, sw);  // with bias: its gradient is the channel sum of dy
	conv.init();
	memcpy(conv.get_weights()->get_data_ptr(), w.data(), w.size() * 4);
	std::vector<float> bias(Cout);
	for (auto& e : bias) e = rnd();
	memcpy(conv.get_bias()->get_data_ptr(), bias.data(), bias.size() * 4);
	conv.to(lten::GPU);
	lten::Tensor Y = conv.forward(X);
	lten::Tensor T = lten::TensorFromBuffer({ (uint64_t)N, (uint64_t)Cout, (uint64_t)Ho, (uint64_t)Wo }, dy.data()).to(lten::GPU);
	Y.backward(&T);
	std::vector<float> y(N * Cout * Ho * Wo, 0), dw(w.size(), 0), dx(x.size(), 0), db(Cout, 0);
	for (int n = 0; n < N; n++) for (int co = 0; co < Cout; co++) for (int p = 0; p < Ho * Wo; p++) {
		y[(n * Cout + co) * Ho * Wo + p] = bias[co];
		db[co] += dy[(n * Cout + co) * Ho * Wo + p];
	}
	for (int n = 0; n < N; n++) for (int co = 0; co < Cout; co++) for (int ho = 0; ho < Ho; ho++) for (int wo = 0; wo < Wo; wo++)
		for (int ci = 0; ci < Cin; ci++) for (int i = 0; i < kh; i++) for (int j = 0; j < kw; j++) {
			const int yy = ho * sh - ph + i, xx = wo * sw - pw + j;
			if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
			const int xi = ((n * Cin + ci) * H + yy) * W + xx, wi = ((co * Cin + ci) * kh + i) * kw + j, yi = ((n * Cout + co) * Ho + ho) * Wo + wo;
			y[yi] += w[wi] * x[xi];
			dw[wi] += dy[yi] * x[xi];
			dx[xi] += dy[yi] * w[wi];
		}
	lten::Tensor Yc = Y.to(lten::CPU);
	const double tol = 1e-4;
	if (Compare((float*)Yc.get_data_ptr(), y.data(), y.size(), tol)) return -1;
	if (Compare(grad_to_host(*conv.get_weights()).data(), dw.data(), dw.size(), tol)) return -2;
	if (Compare(grad_to_host(X).data(), dx.data(), dx.size(), tol)) return -3;
	if (Compare(grad_to_host(*conv.get_bias()).data(), db.data(), db.size(), tol)) return -4;
	return 0;
}

// error behaviour: the same conditions raise the same errors as in l-ten (LTEN_ERR throws lten::ExceptionInfo)
static int error_test()
{
	int caught = 0;
	float buf[64] = { 0 };
	lten::FullyConnected fc(3, 8);
	fc.init();
	fc.to(lten::GPU);
	lten::Tensor two_d = lten::TensorFromBuffer({ 4, 3 }, buf).to(lten::GPU);
	try { fc.forward(two_d); } catch (lten::ExceptionInfo& e) { caught += strstr(e.what(), "at least 3 dimensions") != nullptr; }
	lten::Tensor bad_width = lten::TensorFromBuffer({ 1, 4, 4 }, buf).to(lten::GPU);
	try { fc.forward(bad_width); } catch (lten::ExceptionInfo& e) { caught += strstr(e.what(), "Last dimension must be equal") != nullptr; }
	lten::Tensor on_cpu = lten::TensorFromBuffer({ 1, 4, 3 }, buf);
	try { fc.forward(on_cpu); } catch (lten::ExceptionInfo& e) { caught += strstr(e.what(), "device type or data type") != nullptr; }
	lten::Tensor a = lten::TensorFromBuffer({ 1, 2, 3 }, buf).to(lten::GPU), b = lten::TensorFromBuffer({ 1, 4, 2 }, buf).to(lten::GPU);
	try { a.matmul(b); } catch (lten::ExceptionInfo& e) { caught += strstr(e.what(), "compatiple dimensions") != nullptr; }
	lten::Conv2d conv(1, 2, false, 3, 3);
	conv.init();
	conv.to(lten::GPU);
	try { conv.forward(a); } catch (lten::ExceptionInfo& e) { caught += strstr(e.what(), "exactly 4 dimensions") != nullptr; }
	return caught == 5 ? 0 : -1;
}

// `test_host bench`: the int8 FullyConnected_q forward at 4096^3 as a caller of the layer API sees it, copies included:
// input tensor on the CPU -> to(GPU), forward, result -> to(CPU); and the forward alone on a resident input.  The layer
// (weights, their int8 form) is moved to the GPU once beforehand, as a network is.  Prints one JSON line.
#include <algorithm>
#include <chrono>
#include "../../include/lten_hip.h"
static int api_bench()
{
	const uint64_t M = 4096, K = 4096, N = 4096;
	std::vector<uint8_t> x(M * K), w(N * K);
	unsigned s = 7;
	auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (s >> 16) & 0xFF; };
	for (auto& e : x) e = (uint8_t)rnd();
	for (auto& e : w) e = (uint8_t)(128 + (int)(rnd() % 81) - 40);
	lten::TensorOps ops;
	ops.data_type = lten::UINT8;
	lten::FullyConnected_q fc(K, N, false);
	fc.init();
	fc.train(false);
	memcpy(fc.get_weights()->get_data_ptr(), w.data(), w.size());
	QuantizationParams qi{ 0.02f, 128 }, qw{ 0.02f, 128 }, qo{ 1.0f, 128 };
	fc.set_qparams_in(qi);
	fc.set_qparams_params(&qw, 1);
	fc.set_qparams_out(qo);
	fc.to(lten::GPU);
	lten::Tensor Xc = lten::TensorFromBuffer({ 1, M, K }, x.data(), false, &ops);
	auto now = [] { return std::chrono::steady_clock::now(); };
	auto ms = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) { return std::chrono::duration<double, std::milli>(b - a).count(); };
	double best_api = 1e30, best_resident = 1e30;
	for (int rep = 0; rep < 5; rep++) {
		auto t0 = now();
		lten::Tensor Xg = Xc.to(lten::GPU);
		lten::Tensor Y = fc.forward(Xg).to(lten::CPU);  // the download waits for the product
		best_api = std::min(best_api, ms(t0, now()));
	}
	lten::Tensor Xg = Xc.to(lten::GPU);
	for (int rep = 0; rep < 3; rep++) {
		lten::Tensor warm = fc.forward(Xg);
		lten_hip_sync();
		const int iters = 200;
		auto t0 = now();
		for (int i = 0; i < iters; i++) lten::Tensor Y = fc.forward(Xg);
		lten_hip_sync();
		best_resident = std::min(best_resident, ms(t0, now()) / iters);
	}
	const double ops2 = 2.0 * M * N * K;
	printf("{\"api\": \"lten::Tensor::to + lten::FullyConnected_q::forward\", \"with_copies_ms\": %.3f, \"with_copies_tops\": %.2f, "
	       "\"resident_ms_per_forward\": %.5f, \"resident_tops\": %.1f}\n",
	       best_api, ops2 / (best_api * 1e-3) / 1e12, best_resident, ops2 / (best_resident * 1e-3) / 1e12);
	return 0;
}

int main(int argc, char** argv)
{
	if (argc > 1 && strcmp(argv[1], "bench") == 0) {
		try { return api_bench(); } catch (std::exception& e) { printf("exception: %s\n", e.what()); return 1; }
	}
	struct { const char* name; int (*fn)(); } tests[] = { { "matmul_test", matmul_test }, { "fc_test", fc_test }, { "fc_chain_test", fc_chain_test }, { "mlp_step_test", mlp_step_test }, { "training_test", training_test }, { "conv_training_test", conv_training_test },
		                                                  { "fcq_test", fcq_test }, { "fcq_reload_test", fcq_reload_test }, { "conv_test", conv_test }, { "convq_test", convq_test }, { "error_test", error_test } };
	int failed = 0;
	for (auto& t : tests) {
		printf("running %s\n", t.name);
		fflush(stdout);
		int rc = -100;
		try { rc = t.fn(); } catch (std::exception& e) { printf("  exception: %s\n", e.what()); }
		printf("%s %s (%d)\n", t.name, rc == 0 ? "passed" : "FAILED", rc);
		failed += rc != 0;
	}
	printf("%d of %d tests passed\n", (int)(sizeof(tests) / sizeof(tests[0])) - failed, (int)(sizeof(tests) / sizeof(tests[0])));
	return failed ? 1 : 0;
}
