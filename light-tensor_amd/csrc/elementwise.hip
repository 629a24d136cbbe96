// The element-wise and loss pieces that sit between the GEMMs of an MLP training step, so that the step stays on
// the device: relu / relu_backward (l-ten/layers.cpp:9-67, l-ten/backprop.cpp:2282-2327; gpu_relu, gpu_relu_backward
// in l-ten/math_fns.h:231-234), log_softmax along the last dimension (l-ten/layers.cpp:93-114: l-ten composes it from
// max, sub, exp, sum, div, log) with the collapsed form of its backward chain, nll_loss and its backward
// (l-ten/layers.cpp:212-273, l-ten/backprop.cpp:3975-4040; gpu_nll, gpu_mul), and the leaf-gradient accumulate
// (l-ten/backprop.cpp:246-274, cublasSaxpy).  All of them are one pass over their operands (HBM bound when large,
// launch bound at the sizes of l-ten's networks).
#include "common.h"

#include <algorithm>
#include <cmath>

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

// Rows of at most 32 values: LPR = 16 or 32 lanes per row, 64 / LPR rows per wavefront, a value per lane (a wavefront
// per row of 16 values leaves 48 lanes idle: 1048576 x 16 took 230 us).  The folds over a row's lanes are the last ones
// of the wavefront-wide folds above and the lanes past a row's end hold what those would have added (zero, minus
// infinity), so every sum and maximum has the same bits as in the kernels above.
template <int LPR>
__global__ __launch_bounds__(256) void log_softmax_narrow_kernel(uint64_t rows, int cols, const float* __restrict__ x, float* __restrict__ y)
{
	const int lane = threadIdx.x & 63, sub = lane % LPR;
	const uint64_t row = ((uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / LPR) + lane / LPR;
	const bool live = row < rows && sub < cols;
	const float v = live ? x[row * cols + sub] : -INFINITY;
	float m = v;
#pragma unroll
	for (int o = LPR / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
	float e = live ? expf(v - m) : 0.0f, t = e;
#pragma unroll
	for (int o = 32; o >= LPR; o >>= 1) t += 0.0f;  // the folds over lanes that hold nothing (they turn -0 into +0)
#pragma unroll
	for (int o = LPR / 2; o > 0; o >>= 1) t += __shfl_xor(t, o, 64);
	if (live) y[row * cols + sub] = logf(e / t);
}

// (SCALED: the incoming gradient is alpha times dy, as nll_log_softmax_backward_kernel takes it)
template <int LPR, bool SCALED = false>
__global__ __launch_bounds__(256) void log_softmax_backward_narrow_kernel(uint64_t rows, int cols, const float* __restrict__ y, const float* __restrict__ dy,
                                                                          float* __restrict__ dx, float alpha = 1.0f)
{
	const int lane = threadIdx.x & 63, sub = lane % LPR;
	const uint64_t row = ((uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / LPR) + lane / LPR;
	const bool live = row < rows && sub < cols;
	const float g = live ? (SCALED ? alpha * dy[row * cols + sub] : dy[row * cols + sub]) : 0.0f;
	float t = g;
#pragma unroll
	for (int o = 32; o >= LPR; o >>= 1) t += 0.0f;
#pragma unroll
	for (int o = LPR / 2; o > 0; o >>= 1) t += __shfl_xor(t, o, 64);
	if (live) dx[row * cols + sub] = g - expf(y[row * cols + sub]) * t;
}

// Rows of 256 values and more: a workgroup of T threads per row, which keeps the row in registers (up to R values a
// thread, value c in thread c % T) between the maximum, the sum and the output; rows longer than T * R are read again
// from memory for each of the three.  A wavefront per row walks such a row alone, three times over: 64 x 50257 took
// 391 us, 4096 x 4096 68 us.  Sums: a thread's values in order, the wavefront fold, then the wavefronts in order.
template <int T, int R, bool FITS>
__global__ __launch_bounds__(T) void log_softmax_wide_kernel(uint64_t cols, const float* __restrict__ x, float* __restrict__ y)
{
	__shared__ float part[T / 64];
	const int tid = threadIdx.x;
	const float* xr = x + (uint64_t)blockIdx.x * cols;
	float* yr = y + (uint64_t)blockIdx.x * cols;
	float v[R];
	float m = -INFINITY;
	if (FITS) {
#pragma unroll
		for (int i = 0; i < R; i++) {
			const uint64_t c = (uint64_t)tid + (uint64_t)i * T;
			v[i] = c < cols ? xr[c] : -INFINITY;
			m = fmaxf(m, v[i]);
		}
	} else {
		for (uint64_t c = tid; c < cols; c += T) m = fmaxf(m, xr[c]);
	}
	m = wave_max(m);
	if ((tid & 63) == 0) part[tid >> 6] = m;
	__syncthreads();
	m = part[0];
#pragma unroll
	for (int w = 1; w < T / 64; w++) m = fmaxf(m, part[w]);
	__syncthreads();
	float s = 0.0f;
	if (FITS) {
#pragma unroll
		for (int i = 0; i < R; i++) {
			v[i] = expf(v[i] - m);  // exp(-inf) = 0 past the row's end
			s += v[i];
		}
	} else {
		for (uint64_t c = tid; c < cols; c += T) s += expf(xr[c] - m);
	}
	s = wave_sum(s);
	if ((tid & 63) == 0) part[tid >> 6] = s;
	__syncthreads();
	s = part[0];
#pragma unroll
	for (int w = 1; w < T / 64; w++) s += part[w];
	if (FITS) {
#pragma unroll
		for (int i = 0; i < R; i++) {
			const uint64_t c = (uint64_t)tid + (uint64_t)i * T;
			if (c < cols) yr[c] = logf(v[i] / s);
		}
	} else {
		for (uint64_t c = tid; c < cols; c += T) yr[c] = logf(expf(xr[c] - m) / s);
	}
}

template <int T, int R, bool FITS, bool SCALED = false>
__global__ __launch_bounds__(T) void log_softmax_backward_wide_kernel(uint64_t cols, const float* __restrict__ y, const float* __restrict__ dy,
                                                                      float* __restrict__ dx, float alpha = 1.0f)
{
	__shared__ float part[T / 64];
	const int tid = threadIdx.x;
	const float* yr = y + (uint64_t)blockIdx.x * cols;
	const float* gr = dy + (uint64_t)blockIdx.x * cols;
	float* dr = dx + (uint64_t)blockIdx.x * cols;
	float g[R];
	float s = 0.0f;
	if (FITS) {
#pragma unroll
		for (int i = 0; i < R; i++) {
			const uint64_t c = (uint64_t)tid + (uint64_t)i * T;
			g[i] = c < cols ? (SCALED ? alpha * gr[c] : gr[c]) : 0.0f;
			s += g[i];
		}
	} else {
		for (uint64_t c = tid; c < cols; c += T) s += SCALED ? alpha * gr[c] : gr[c];
	}
	s = wave_sum(s);
	if ((tid & 63) == 0) part[tid >> 6] = s;
	__syncthreads();
	s = part[0];
#pragma unroll
	for (int w = 1; w < T / 64; w++) s += part[w];
	if (FITS) {
#pragma unroll
		for (int i = 0; i < R; i++) {
			const uint64_t c = (uint64_t)tid + (uint64_t)i * T;
			if (c < cols) dr[c] = g[i] - expf(yr[c]) * s;
		}
	} else {
		for (uint64_t c = tid; c < cols; c += T) dr[c] = (SCALED ? alpha * gr[c] : gr[c]) - expf(yr[c]) * s;
	}
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

// The same sum for long arrays (the log-probabilities of a large batch over a large vocabulary: one workgroup took 9.6
// ms over 32768 x 1000 values): workgroup b sums a contiguous share the way the kernel above sums the whole array and
// leaves it in partial[b]; a second launch of the kernel below adds the shares in index order and scales.
__global__ __launch_bounds__(1024) void nll_loss_partial_kernel(const float* __restrict__ input, const float* __restrict__ target, float* __restrict__ partial,
                                                                uint64_t len, uint64_t share)
{
	__shared__ float part[16];
	const uint64_t begin = (uint64_t)blockIdx.x * share, end = begin + share < len ? begin + share : len;
	float s = 0.0f;
	for (uint64_t i = begin + threadIdx.x; i < end; i += 1024) s += input[i] * target[i];
	s = wave_sum(s);
	if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
	__syncthreads();
	if (threadIdx.x == 0) {
		float tot = 0.0f;
#pragma unroll
		for (int w = 0; w < 16; w++) tot += part[w];
		partial[blockIdx.x] = tot;
	}
}

__global__ __launch_bounds__(64) void nll_loss_finish_kernel(const float* __restrict__ partial, int count, float* __restrict__ loss, float scale)
{
	if (threadIdx.x != 0) return;
	float tot = 0.0f;
	for (int b = 0; b < count; b++) tot += partial[b];
	*loss = tot * scale;
}

// log_softmax, nll_loss and (GRAD) the gradient of the loss with respect to the logits for a small batch of narrow
// rows (rows <= 1024, cols <= 16) in one launch of one workgroup: a thread per row, the row in registers.  The separate
// kernels fold a row across a wavefront by lane exchanges; with the row in one thread the same sums are taken in the
// same order (pairs 8 apart, then 4, 2, 1: what the exchange tree leaves in lane 0 when all lanes past the row hold
// zeros), so the log-probabilities and the gradient are bit-identical to theirs, and the loss is summed from an LDS copy
// of the log-probabilities exactly as nll_loss_kernel sums it from memory.  One workgroup because a hand-over between
// workgroups (release fence, arrival counter) costs more on this part than the whole computation.
__device__ __forceinline__ float tree_sum16(float (&v)[16])
{
	float t[16];
#pragma unroll
	for (int i = 0; i < 16; i++) t[i] = v[i];
#pragma unroll
	for (int o = 8; o > 0; o >>= 1)
#pragma unroll
		for (int i = 0; i < o; i++) t[i] = t[i] + t[i + o];
	return t[0];
}

template <bool GRAD>
__global__ __launch_bounds__(1024) void loss_rows_kernel(int rows, int cols, const float* __restrict__ x, const float* __restrict__ target, float alpha,
                                                         float* __restrict__ y, float* __restrict__ loss, float loss_scale, float* __restrict__ dx)
{
	__shared__ float logp[16384];
	__shared__ float part[16];
	const int r = threadIdx.x;
	if (r < rows) {
		float xv[16], tv[16];
#pragma unroll
		for (int c = 0; c < 16; c++) {
			xv[c] = c < cols ? x[r * cols + c] : -INFINITY;
			tv[c] = (GRAD && c < cols) ? target[r * cols + c] : 0.0f;
		}
		float m = -INFINITY;
#pragma unroll
		for (int c = 0; c < 16; c++) m = fmaxf(m, xv[c]);
		float e[16];
#pragma unroll
		for (int c = 0; c < 16; c++) e[c] = c < cols ? expf(xv[c] - m) : 0.0f;
		const float s = tree_sum16(e);
		float lp[16];
#pragma unroll
		for (int c = 0; c < 16; c++) {
			lp[c] = logf(e[c] / s);
			if (c < cols) {
				y[r * cols + c] = lp[c];
				logp[r * cols + c] = lp[c];
			}
		}
		if (GRAD) {
			float dy[16];
#pragma unroll
			for (int c = 0; c < 16; c++) dy[c] = c < cols ? alpha * tv[c] : 0.0f;
			const float sdy = tree_sum16(dy);
#pragma unroll
			for (int c = 0; c < 16; c++)
				if (c < cols) dx[r * cols + c] = dy[c] - expf(lp[c]) * sdy;
		}
	}
	__syncthreads();
	const int len = rows * cols;
	float acc = 0.0f;
	for (int i = threadIdx.x; i < len; i += 1024) acc += logp[i] * target[i];
	acc = wave_sum(acc);
	if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
	__syncthreads();
	if (threadIdx.x == 0) {
		float tot = 0.0f;
#pragma unroll
		for (int w = 0; w < 16; w++) tot += part[w];
		*loss = tot * loss_scale;
	}
}

// nll_backward (dy = alpha * target, gpu_mul) and the backward of log_softmax in one pass; the same operations per
// element as scale_kernel followed by log_softmax_backward_kernel.
__global__ __launch_bounds__(256) void nll_log_softmax_backward_kernel(uint64_t rows, uint64_t cols, const float* __restrict__ y,
                                                                       const float* __restrict__ target, float alpha, float* __restrict__ dx)
{
	const int lane = threadIdx.x & 63;
	const uint64_t row = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= rows) return;
	float s = 0.0f;
	for (uint64_t c = lane; c < cols; c += 64) s += alpha * target[row * cols + c];
	s = wave_sum(s);
	for (uint64_t c = lane; c < cols; c += 64) dx[row * cols + c] = alpha * target[row * cols + c] - expf(y[row * cols + c]) * s;
}

// SGDOptimizer::step for one tensor (l-ten/optimizer.cpp:52-57; gpu_sgd_step, l-ten/math_fns.h:186): the gradient
// buffer receives the decayed gradient, as in l-ten.  Every product and sum rounded on its own, in l-ten's order.
__global__ __launch_bounds__(256) void sgd_step_kernel(float* __restrict__ w, float* __restrict__ g, float* __restrict__ v, uint64_t n, float mo,
                                                       float wd, float lr)
{
#pragma clang fp contract(off)
	const float one_minus_mo = 1.0f - mo;
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
		const float gd = wd * w[i] + g[i];
		const float vel = v[i] * mo + one_minus_mo * gd;
		g[i] = gd;
		v[i] = vel;
		w[i] = w[i] - (vel * lr);
	}
}

// AdamOptimizer::step for one tensor (l-ten/optimizer.cpp:139-155): l-ten's eight element-wise launches (axpby, mul,
// axpby, mul, powx, add, div, axpy) as one pass, same operations in the same order per element.
__global__ __launch_bounds__(256) void adam_step_kernel(float* __restrict__ w, const float* __restrict__ g, float* __restrict__ v, float* __restrict__ s,
                                                        uint64_t n, float a1, float beta1, float a2, float beta2, float inv_bc2, float step)
{
#pragma clang fp contract(off)
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
		const float gi = g[i];
		const float vi = a1 * gi + beta1 * v[i];
		const float si = a2 * (gi * gi) + beta2 * s[i];
		float t = inv_bc2 * si;
		t = powf(t, 0.5f);
		t = 1.0e-8f + t;
		t = vi / t;
		v[i] = vi;
		s[i] = si;
		w[i] = (step == 1.0f) ? w[i] + t : w[i] + step * t;
	}
}

static unsigned grid_for(uint64_t n) { return (unsigned)std::min<uint64_t>(ceil_div(n, 256), 256 * 16); }

// Channel sums of an NCHW gradient: db[c] (+)= sum over n, h, w of dy[n][c][h][w] — what the backward pass of the
// broadcast add leaves in the bias of a convolution (l-ten/conv2d.cpp:189-192 adds the bias {1, C, 1, 1} as a
// tensor op; l-ten/backprop.cpp:605-690 sums the top gradient over the broadcast dimensions).  Workgroup (c, s) adds
// slice s of the images of channel c; a second launch adds the slices in slice order.  The partial sums live in a
// small device array of the library.
constexpr int CHANNEL_SUM_SLOTS = 4096;
static __device__ float g_channel_partial[CHANNEL_SUM_SLOTS];

__global__ __launch_bounds__(256) void channel_sum_partial_kernel(const float* __restrict__ dy, int N, int C, int64_t HW, int slices, float* __restrict__ partial)
{
	__shared__ float part[4];
	const int c = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
	// the slice's share of the N * HW values of channel c, taken in runs of 256 consecutive values; (n, hw) advance
	// by a fixed step without a division per element
	const int64_t step = (int64_t)slices * 256, step_n = step / HW, step_hw = step % HW;
	int64_t n = ((int64_t)s * 256 + tid) / HW, hw = ((int64_t)s * 256 + tid) % HW;
	float sum = 0.0f;
	while (n < N) {
		sum += dy[(n * C + c) * HW + hw];
		n += step_n;
		hw += step_hw;
		if (hw >= HW) { hw -= HW; n++; }
	}
#pragma unroll
	for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off);
	if ((tid & 63) == 0) part[tid >> 6] = sum;
	__syncthreads();
	if (tid == 0) partial[c * slices + s] = ((part[0] + part[1]) + part[2]) + part[3];
}

__global__ __launch_bounds__(256) void channel_sum_final_kernel(const float* __restrict__ partial, int C, int slices, float* __restrict__ db, int accumulate)
{
	const int c = blockIdx.x * 256 + threadIdx.x;
	if (c >= C) return;
	// (eight loads in flight at a time, the additions in slice order)
	float sum = 0.0f;
	int s = 0;
	for (; s + 8 <= slices; s += 8) {
		float v[8];
#pragma unroll
		for (int j = 0; j < 8; j++) v[j] = partial[c * slices + s + j];
#pragma unroll
		for (int j = 0; j < 8; j++) sum += v[j];
	}
	for (; s < slices; s++) sum += partial[c * slices + s];
	db[c] = accumulate ? db[c] + sum : sum;
}

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
	if (cols <= 16 && rows >= 1024) log_softmax_narrow_kernel<16><<<dim3((unsigned)ceil_div(rows, 16)), dim3(256), 0, stream()>>>(rows, (int)cols, x, y);
	else if (cols <= 32 && rows >= 1024) log_softmax_narrow_kernel<32><<<dim3((unsigned)ceil_div(rows, 8)), dim3(256), 0, stream()>>>(rows, (int)cols, x, y);
	else if (cols >= 256 && cols <= 2048) log_softmax_wide_kernel<256, 8, true><<<dim3((unsigned)rows), dim3(256), 0, stream()>>>(cols, x, y);
	else if (cols > 2048 && cols <= 8192) log_softmax_wide_kernel<256, 32, true><<<dim3((unsigned)rows), dim3(256), 0, stream()>>>(cols, x, y);
	else if (cols > 8192 && cols <= 65536) log_softmax_wide_kernel<1024, 64, true><<<dim3((unsigned)rows), dim3(1024), 0, stream()>>>(cols, x, y);
	else if (cols > 65536) log_softmax_wide_kernel<1024, 1, false><<<dim3((unsigned)rows), dim3(1024), 0, stream()>>>(cols, x, y);
	else log_softmax_kernel<<<dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, stream()>>>(rows, cols, x, y);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_log_softmax_backward_f32(uint64_t rows, uint64_t cols, const float* y, const float* dy, float* dx)
{
	if (rows == 0 || cols == 0) return 0;
	LTEN_HIP_REQUIRE(y && dy && dx, "log_softmax_backward: null pointer");
	LTEN_HIP_REQUIRE(ceil_div(rows, 4) < (1ull << 31), "log_softmax_backward: too many rows");
	if (cols <= 16 && rows >= 1024) log_softmax_backward_narrow_kernel<16><<<dim3((unsigned)ceil_div(rows, 16)), dim3(256), 0, stream()>>>(rows, (int)cols, y, dy, dx);
	else if (cols <= 32 && rows >= 1024) log_softmax_backward_narrow_kernel<32><<<dim3((unsigned)ceil_div(rows, 8)), dim3(256), 0, stream()>>>(rows, (int)cols, y, dy, dx);
	else if (cols >= 256 && cols <= 2048) log_softmax_backward_wide_kernel<256, 8, true><<<dim3((unsigned)rows), dim3(256), 0, stream()>>>(cols, y, dy, dx);
	else if (cols > 2048 && cols <= 8192) log_softmax_backward_wide_kernel<256, 32, true><<<dim3((unsigned)rows), dim3(256), 0, stream()>>>(cols, y, dy, dx);
	else if (cols > 8192 && cols <= 65536) log_softmax_backward_wide_kernel<1024, 64, true><<<dim3((unsigned)rows), dim3(1024), 0, stream()>>>(cols, y, dy, dx);
	else if (cols > 65536) log_softmax_backward_wide_kernel<1024, 1, false><<<dim3((unsigned)rows), dim3(1024), 0, stream()>>>(cols, y, dy, dx);
	else log_softmax_backward_kernel<<<dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, stream()>>>(rows, cols, y, dy, dx);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_sgd_step_f32(float* weight, float* weight_grad, float* velocity, uint64_t numels, float mo, float wd, float lr)
{
	if (numels == 0) return 0;
	LTEN_HIP_REQUIRE(weight && weight_grad && velocity, "sgd_step: null pointer");
	sgd_step_kernel<<<dim3(grid_for(numels)), dim3(256), 0, stream()>>>(weight, weight_grad, velocity, numels, mo, wd, lr);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_adam_step_f32(float* weight, const float* weight_grad, float* v_dw, float* s_dw, uint64_t numels, float lr,
                           float beta1, float beta2, uint64_t iteration)
{
	if (numels == 0) return 0;
	LTEN_HIP_REQUIRE(weight && weight_grad && v_dw && s_dw && iteration > 0, "adam_step: null pointer or iteration 0");
	// l-ten/optimizer.cpp:136-137, :139-155: host scalars exactly as l-ten forms them
	const float bc1 = 1.0f - powf(beta1, static_cast<float>(iteration));
	const float bc2 = 1.0f - powf(beta2, static_cast<float>(iteration));
	adam_step_kernel<<<dim3(grid_for(numels)), dim3(256), 0, stream()>>>(weight, weight_grad, v_dw, s_dw, numels, 1.0f - beta1, beta1, 1.0f - beta2,
	                                                                     beta2, 1.0f / bc2, -(1.0f / bc1) * lr);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_nll_loss_f32(const float* input, const float* target, float* loss, uint64_t len, uint64_t batches)
{
	LTEN_HIP_REQUIRE(loss != nullptr && batches > 0, "nll_loss: null loss pointer or zero batch");
	LTEN_HIP_REQUIRE(len == 0 || (input && target), "nll_loss: null pointer");
	// (up to 65536 values one workgroup: the order of that sum is the one the one-launch loss kernels reproduce)
	constexpr uint64_t SHARE = 32768;
	float* partial = len > 65536 ? static_cast<float*>(library_scratch(4096 * sizeof(float))) : nullptr;
	if (partial != nullptr) {
		const uint64_t share = std::max<uint64_t>(SHARE, (ceil_div(len, 2048) + 1023) / 1024 * 1024);  // at most 2048 shares, whole rounds of the workgroup
		const unsigned count = (unsigned)ceil_div(len, share);
		nll_loss_partial_kernel<<<dim3(count), dim3(1024), 0, stream()>>>(input, target, partial, len, share);
		LTEN_HIP_LAUNCH_CHECK();
		nll_loss_finish_kernel<<<dim3(1), dim3(64), 0, stream()>>>(partial, (int)count, loss, -1.0f / (float)batches);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	nll_loss_kernel<<<dim3(1), dim3(1024), 0, stream()>>>(input, target, loss, len, -1.0f / (float)batches);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

static bool loss_rows_fits(uint64_t rows, uint64_t cols) { return rows >= 1 && rows <= 1024 && cols >= 1 && cols <= 16; }

int lten_hip_log_softmax_nll_loss_f32(uint64_t rows, uint64_t cols, const float* x, const float* target, float* y, float* loss)
{
	LTEN_HIP_REQUIRE(loss != nullptr && rows > 0, "log_softmax_nll_loss: null loss pointer or zero batch");
	LTEN_HIP_REQUIRE(cols == 0 || (x && target && y), "log_softmax_nll_loss: null pointer");
	if (!loss_rows_fits(rows, cols)) {  // the two launches it stands for
		if (int rc = lten_hip_log_softmax_f32(rows, cols, x, y)) return rc;
		return lten_hip_nll_loss_f32(y, target, loss, rows * cols, rows);
	}
	set_kernel_name("loss_rows");
	loss_rows_kernel<false><<<dim3(1), dim3(1024), 0, stream()>>>((int)rows, (int)cols, x, target, 0.0f, y, loss, -1.0f / (float)rows, nullptr);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_log_softmax_nll_loss_grad_f32(uint64_t rows, uint64_t cols, const float* x, const float* target, float alpha, float* y,
                                           float* loss, float* dx)
{
	LTEN_HIP_REQUIRE(loss != nullptr && rows > 0, "log_softmax_nll_loss_grad: null loss pointer or zero batch");
	LTEN_HIP_REQUIRE(cols == 0 || (x && target && y && dx), "log_softmax_nll_loss_grad: null pointer");
	if (!loss_rows_fits(rows, cols)) {  // the launches it stands for
		if (int rc = lten_hip_log_softmax_nll_loss_f32(rows, cols, x, target, y, loss)) return rc;
		return lten_hip_nll_log_softmax_backward_f32(rows, cols, y, target, alpha, dx);
	}
	set_kernel_name("loss_rows_grad");
	loss_rows_kernel<true><<<dim3(1), dim3(1024), 0, stream()>>>((int)rows, (int)cols, x, target, alpha, y, loss, -1.0f / (float)rows, dx);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_nll_log_softmax_backward_f32(uint64_t rows, uint64_t cols, const float* y, const float* target, float alpha, float* dx)
{
	if (rows == 0 || cols == 0) return 0;
	LTEN_HIP_REQUIRE(y && target && dx, "nll_log_softmax_backward: null pointer");
	// the forms of lten_hip_log_softmax_backward_f32 for narrow and wide rows, fed alpha * target
	if (cols <= 16 && rows >= 1024) log_softmax_backward_narrow_kernel<16, true><<<dim3((unsigned)ceil_div(rows, 16)), dim3(256), 0, stream()>>>(rows, (int)cols, y, target, dx, alpha);
	else if (cols <= 32 && rows >= 1024) log_softmax_backward_narrow_kernel<32, true><<<dim3((unsigned)ceil_div(rows, 8)), dim3(256), 0, stream()>>>(rows, (int)cols, y, target, dx, alpha);
	else if (cols >= 256 && cols <= 2048) log_softmax_backward_wide_kernel<256, 8, true, true><<<dim3((unsigned)rows), dim3(256), 0, stream()>>>(cols, y, target, dx, alpha);
	else if (cols > 2048 && cols <= 8192) log_softmax_backward_wide_kernel<256, 32, true, true><<<dim3((unsigned)rows), dim3(256), 0, stream()>>>(cols, y, target, dx, alpha);
	else if (cols > 8192 && cols <= 65536) log_softmax_backward_wide_kernel<1024, 64, true, true><<<dim3((unsigned)rows), dim3(1024), 0, stream()>>>(cols, y, target, dx, alpha);
	else if (cols > 65536) log_softmax_backward_wide_kernel<1024, 1, false, true><<<dim3((unsigned)rows), dim3(1024), 0, stream()>>>(cols, y, target, dx, alpha);
	else nll_log_softmax_backward_kernel<<<dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, stream()>>>(rows, cols, y, target, alpha, dx);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_conv2d_bias_grad_f32(uint64_t N, uint64_t C, uint64_t HW, const float* dy, float* db, int accumulate)
{
	if (C == 0) return 0;
	LTEN_HIP_REQUIRE(db != nullptr, "conv2d_bias_grad: db is null");
	LTEN_HIP_REQUIRE(N * HW == 0 || dy != nullptr, "conv2d_bias_grad: dy is null");
	LTEN_HIP_REQUIRE(C <= CHANNEL_SUM_SLOTS && N < (1ull << 31) && HW < (1ull << 40), "conv2d_bias_grad: more than %d channels", CHANNEL_SUM_SLOTS);
	if (N * HW == 0) return accumulate ? 0 : lten_hip_zero(db, C * sizeof(float));  // nothing to sum
	const uint64_t runs = ceil_div(N * HW, 256);
	const int slices = (int)std::max<uint64_t>(1, std::min<uint64_t>(std::min<uint64_t>(CHANNEL_SUM_SLOTS / C, 64), runs));
	float* partial = nullptr;
	LTEN_HIP_CHECK(hipGetSymbolAddress(reinterpret_cast<void**>(&partial), HIP_SYMBOL(g_channel_partial)));
	set_kernel_name("channel_sum");
	channel_sum_partial_kernel<<<dim3((unsigned)C, (unsigned)slices), dim3(256), 0, stream()>>>(dy, (int)N, (int)C, (int64_t)HW, slices, partial);
	LTEN_HIP_LAUNCH_CHECK();
	channel_sum_final_kernel<<<dim3((unsigned)ceil_div(C, 256)), dim3(256), 0, stream()>>>(partial, (int)C, slices, db, accumulate);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // extern "C"
