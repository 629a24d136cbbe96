// The element-wise and loss pieces that sit between the GEMMs of an MLP training step, so that the step stays on
// the device: relu / relu_backward (l-ten/layers.cpp:9-67, l-ten/backprop.cpp:2282-2327; gpu_relu, gpu_relu_backward
// in l-ten/math_fns.h:231-234), log_softmax along the last dimension (l-ten/layers.cpp:93-114: l-ten composes it from
// max, sub, exp, sum, div, log) with the collapsed form of its backward chain, nll_loss and its backward
// (l-ten/layers.cpp:212-273, l-ten/backprop.cpp:3975-4040; gpu_nll, gpu_mul), and the leaf-gradient accumulate
// (l-ten/backprop.cpp:246-274, cublasSaxpy).  All of them are one pass over their operands (HBM bound when large,
// launch bound at the sizes of l-ten's networks).
#include "common.h"

#include <algorithm>

namespace lten_hip {

__global__ __launch_bounds__(256) void relu_kernel(const float* __restrict__ src, float* __restrict__ dst, uint64_t n)
{
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
		const float v = src[i];
		dst[i] = v > 0 ? v : 0.0f;
	}
}

__global__ __launch_bounds__(256) void relu_backward_kernel(const float* __restrict__ top, const float* __restrict__ input,
                                                            float* __restrict__ bottom, uint64_t n)
{
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256)
		bottom[i] = input[i] > 0 ? top[i] : 0.0f;
}

// y = alpha * x (gpu_mul(N, alpha, A, B)) or y += alpha * x (saxpy)
template <bool ACCUMULATE>
__global__ __launch_bounds__(256) void scale_kernel(uint64_t n, float alpha, const float* __restrict__ x, float* __restrict__ y)
{
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
		const float v = alpha * x[i];
		y[i] = ACCUMULATE ? y[i] + v : v;
	}
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
	return v;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
	return v;
}

// One wavefront per row: max, sum of exp(x - max), then log(exp(x - max) / sum) as l-ten's chain of ops writes it.
__global__ __launch_bounds__(256) void log_softmax_kernel(uint64_t rows, uint64_t cols, const float* __restrict__ x, float* __restrict__ y)
{
	const int lane = threadIdx.x & 63;
	const uint64_t row = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= rows) return;
	const float* xr = x + row * cols;
	float m = -INFINITY;
	for (uint64_t c = lane; c < cols; c += 64) m = fmaxf(m, xr[c]);
	m = wave_max(m);
	float s = 0.0f;
	for (uint64_t c = lane; c < cols; c += 64) s += expf(xr[c] - m);
	s = wave_sum(s);
	for (uint64_t c = lane; c < cols; c += 64) y[row * cols + c] = logf(expf(xr[c] - m) / s);
}

// dx = dy - exp(y) * sum_j dy_j: what l-ten's backward functions of log, div, sum, exp, sub and max add up to.
__global__ __launch_bounds__(256) void log_softmax_backward_kernel(uint64_t rows, uint64_t cols, const float* __restrict__ y,
                                                                   const float* __restrict__ dy, float* __restrict__ dx)
{
	const int lane = threadIdx.x & 63;
	const uint64_t row = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= rows) return;
	float s = 0.0f;
	for (uint64_t c = lane; c < cols; c += 64) s += dy[row * cols + c];
	s = wave_sum(s);
	for (uint64_t c = lane; c < cols; c += 64) dx[row * cols + c] = dy[row * cols + c] - expf(y[row * cols + c]) * s;
}

// loss = (sum_i input[i] * target[i]) * (-1 / batch): one workgroup, lanes stride the array, fixed-order tree.
__global__ __launch_bounds__(1024) void nll_loss_kernel(const float* __restrict__ input, const float* __restrict__ target, float* __restrict__ loss,
                                                        uint64_t len, float scale)
{
	__shared__ float part[16];
	float s = 0.0f;
	for (uint64_t i = threadIdx.x; i < len; i += 1024) s += input[i] * target[i];
	s = wave_sum(s);
	if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
	__syncthreads();
	if (threadIdx.x == 0) {
		float tot = 0.0f;
#pragma unroll
		for (int w = 0; w < 16; w++) tot += part[w];
		*loss = tot * scale;
	}
}

static unsigned grid_for(uint64_t n) { return (unsigned)std::min<uint64_t>(ceil_div(n, 256), 256 * 16); }

}  // namespace lten_hip

using namespace lten_hip;

extern "C" {

int lten_hip_relu_f32(float* dst, const float* src, uint64_t len)
{
	if (len == 0) return 0;
	LTEN_HIP_REQUIRE(dst && src, "relu: null pointer");
	relu_kernel<<<dim3(grid_for(len)), dim3(256), 0, stream()>>>(src, dst, len);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_relu_backward_f32(float* bottom, const float* top, const float* input, uint64_t len)
{
	if (len == 0) return 0;
	LTEN_HIP_REQUIRE(bottom && top && input, "relu_backward: null pointer");
	relu_backward_kernel<<<dim3(grid_for(len)), dim3(256), 0, stream()>>>(top, input, bottom, len);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_scale_f32(uint64_t n, float alpha, const float* x, float* y)
{
	if (n == 0) return 0;
	LTEN_HIP_REQUIRE(x && y, "scale: null pointer");
	scale_kernel<false><<<dim3(grid_for(n)), dim3(256), 0, stream()>>>(n, alpha, x, y);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_axpy_f32(uint64_t n, float alpha, const float* x, float* y)
{
	if (n == 0) return 0;
	LTEN_HIP_REQUIRE(x && y, "axpy: null pointer");
	scale_kernel<true><<<dim3(grid_for(n)), dim3(256), 0, stream()>>>(n, alpha, x, y);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_log_softmax_f32(uint64_t rows, uint64_t cols, const float* x, float* y)
{
	if (rows == 0 || cols == 0) return 0;
	LTEN_HIP_REQUIRE(x && y, "log_softmax: null pointer");
	LTEN_HIP_REQUIRE(ceil_div(rows, 4) < (1ull << 31), "log_softmax: too many rows");
	log_softmax_kernel<<<dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, stream()>>>(rows, cols, x, y);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_log_softmax_backward_f32(uint64_t rows, uint64_t cols, const float* y, const float* dy, float* dx)
{
	if (rows == 0 || cols == 0) return 0;
	LTEN_HIP_REQUIRE(y && dy && dx, "log_softmax_backward: null pointer");
	LTEN_HIP_REQUIRE(ceil_div(rows, 4) < (1ull << 31), "log_softmax_backward: too many rows");
	log_softmax_backward_kernel<<<dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, stream()>>>(rows, cols, y, dy, dx);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_nll_loss_f32(const float* input, const float* target, float* loss, uint64_t len, uint64_t batches)
{
	LTEN_HIP_REQUIRE(loss != nullptr && batches > 0, "nll_loss: null loss pointer or zero batch");
	LTEN_HIP_REQUIRE(len == 0 || (input && target), "nll_loss: null pointer");
	nll_loss_kernel<<<dim3(1), dim3(1024), 0, stream()>>>(input, target, loss, len, -1.0f / (float)batches);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // extern "C"
