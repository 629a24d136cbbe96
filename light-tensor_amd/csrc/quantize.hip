// Quantize / Dequantize / GetMinMax of l-ten/utils.cpp:198-286 on the device, so that the tensors entering and leaving
// the quantized layers do not have to travel to the host: q = round(zero_point + x / scale) clamped (uint8: [0, 255];
// int: the float images of INT_MIN / INT_MAX), x = scale * (q - zero_point), and the minimum / maximum that
// ComputeQuantizationParams (host arithmetic on two floats, left to the caller) starts from.  The float operations
// are written one by one as l-ten's build executes them (divide, add, compare-selects, round half away from zero):
// the results are bit-exact with the CPU code.
#include "common.h"

#include <algorithm>

namespace lten_hip {

__global__ __launch_bounds__(256) void quantize_u8_kernel(const float* __restrict__ data, uint8_t* __restrict__ q, uint64_t len, float scale, float zp)
{
#pragma clang fp contract(off)
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < len; i += (uint64_t)gridDim.x * 256) {
		float val = zp + data[i] / scale;
		val = (val < 255.f) ? val : 255.f;  // std::min(255.f, val): NaN becomes 255
		val = (0.f < val) ? val : 0.f;      // std::max(0.f, val)
		q[i] = (uint8_t)roundf(val);
	}
}

__global__ __launch_bounds__(256) void quantize_i32_kernel(const float* __restrict__ data, int32_t* __restrict__ q, uint64_t len, float scale, float zp)
{
#pragma clang fp contract(off)
	const float lowest = -2147483648.0f, highest = 2147483648.0f;  // (float)INT_MAX rounds up to 2^31
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < len; i += (uint64_t)gridDim.x * 256) {
		float val = zp + data[i] / scale;
		val = (val < highest) ? val : highest;
		val = (lowest < val) ? val : lowest;
		const float r = roundf(val);
		// x86's float -> int conversion gives 0x80000000 for what does not fit
		q[i] = (r >= -2147483648.0f && r < 2147483648.0f) ? (int32_t)r : (int32_t)0x80000000u;
	}
}

__global__ __launch_bounds__(256) void dequantize_u8_kernel(float* __restrict__ data, const uint8_t* __restrict__ q, uint64_t len, float scale, int zp)
{
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < len; i += (uint64_t)gridDim.x * 256)
		data[i] = scale * (float)((int)q[i] - zp);
}

// Partial and final results of the minimum / maximum search.  One search at a time per device (calls on the
// library's stream are ordered; the host call below waits for its result).
constexpr int MINMAX_BLOCKS = 512;
__device__ float g_minmax_partial[2 * MINMAX_BLOCKS];
__device__ float g_minmax_result[2];

// l-ten's loop starts from data[0] and replaces on strict comparisons, so NaN elements are skipped unless the first
// element is one (then both results are NaN); fminf / fmaxf skip NaN the same way.
__global__ __launch_bounds__(256) void minmax_partial_kernel(const float* __restrict__ data, uint64_t len)
{
	__shared__ float slo[4], shi[4];
	float lo = INFINITY, hi = -INFINITY;
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < len; i += (uint64_t)gridDim.x * 256) {
		const float v = data[i];
		lo = fminf(lo, v);
		hi = fmaxf(hi, v);
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) {
		lo = fminf(lo, __shfl_xor(lo, o, 64));
		hi = fmaxf(hi, __shfl_xor(hi, o, 64));
	}
	if ((threadIdx.x & 63) == 0) { slo[threadIdx.x >> 6] = lo; shi[threadIdx.x >> 6] = hi; }
	__syncthreads();
	if (threadIdx.x == 0) {
		g_minmax_partial[2 * blockIdx.x] = fminf(fminf(slo[0], slo[1]), fminf(slo[2], slo[3]));
		g_minmax_partial[2 * blockIdx.x + 1] = fmaxf(fmaxf(shi[0], shi[1]), fmaxf(shi[2], shi[3]));
	}
}

__global__ __launch_bounds__(64) void minmax_final_kernel(const float* __restrict__ data, int blocks)
{
	float lo = INFINITY, hi = -INFINITY;
	for (int b = threadIdx.x; b < blocks; b += 64) {
		lo = fminf(lo, g_minmax_partial[2 * b]);
		hi = fmaxf(hi, g_minmax_partial[2 * b + 1]);
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) {
		lo = fminf(lo, __shfl_xor(lo, o, 64));
		hi = fmaxf(hi, __shfl_xor(hi, o, 64));
	}
	if (threadIdx.x == 0) {
		const float first = data[0];
		const bool first_nan = first != first;
		// every element NaN except none compared: with a non-NaN first element the loop's start values are data[0]
		g_minmax_result[0] = first_nan ? first : lo;
		g_minmax_result[1] = first_nan ? first : hi;
	}
}

static unsigned grid_for(uint64_t n) { return (unsigned)std::min<uint64_t>(ceil_div(n, 256), 256 * 16); }

}  // namespace lten_hip

using namespace lten_hip;

extern "C" {

int lten_hip_quantize_u8(const float* data, uint8_t* q_data, uint64_t len, const lten_hip_qparams* qp)
{
	LTEN_HIP_REQUIRE(qp != nullptr, "quantize: qparams is null");
	if (len == 0) return 0;
	LTEN_HIP_REQUIRE(data && q_data, "quantize: null pointer");
	quantize_u8_kernel<<<dim3(grid_for(len)), dim3(256), 0, stream()>>>(data, q_data, len, qp->scale, (float)qp->zero_point);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_quantize_i32(const float* data, int32_t* q_data, uint64_t len, const lten_hip_qparams* qp)
{
	LTEN_HIP_REQUIRE(qp != nullptr, "quantize: qparams is null");
	if (len == 0) return 0;
	LTEN_HIP_REQUIRE(data && q_data, "quantize: null pointer");
	quantize_i32_kernel<<<dim3(grid_for(len)), dim3(256), 0, stream()>>>(data, q_data, len, qp->scale, (float)qp->zero_point);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_dequantize_u8(float* data, const uint8_t* q_data, uint64_t len, const lten_hip_qparams* qp)
{
	LTEN_HIP_REQUIRE(qp != nullptr, "dequantize: qparams is null");
	if (len == 0) return 0;
	LTEN_HIP_REQUIRE(data && q_data, "dequantize: null pointer");
	dequantize_u8_kernel<<<dim3(grid_for(len)), dim3(256), 0, stream()>>>(data, q_data, len, qp->scale, (int)qp->zero_point);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_get_min_max(const float* data, uint64_t len, float* min_val, float* max_val)
{
	// l-ten/utils.cpp:203-206
	LTEN_HIP_REQUIRE(data && min_val && max_val && len > 0, "Invalid argument");
	LTEN_HIP_REQUIRE(!capturing(), "lten_hip_get_min_max: not allowed between lten_hip_graph_begin and lten_hip_graph_end");
	const int blocks = (int)std::min<uint64_t>(ceil_div(len, 256), MINMAX_BLOCKS);
	minmax_partial_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(data, len);
	LTEN_HIP_LAUNCH_CHECK();
	minmax_final_kernel<<<dim3(1), dim3(64), 0, stream()>>>(data, blocks);
	LTEN_HIP_LAUNCH_CHECK();
	float host[2];
	LTEN_HIP_CHECK(hipMemcpyFromSymbolAsync(host, HIP_SYMBOL(g_minmax_result), sizeof(host), 0, hipMemcpyDeviceToHost, stream()));
	LTEN_HIP_CHECK(hipStreamSynchronize(stream()));
	*min_val = host[0];
	*max_val = host[1];
	return 0;
}

}  // extern "C"
