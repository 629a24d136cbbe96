// Calibration kernels for the roofline figures, built into a library of their own (liblten_hip_measure.so): they are
// no part of the drop-in surface.  The MFMA issue rate this part actually sustains with no memory traffic at all, and
// the HBM rate of a plain copy.  l-ten has no counterpart; these exist so that reported fractions can be stated
// against measured ceilings as well as against the published peaks, and so that profiler byte counters can be scaled
// by a kernel whose traffic is known.  Everything runs on the null stream.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/lten_hip_measure.h"

namespace lten_measure {

static thread_local char g_error[256] = "";
static void set_error(const char* fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_error, sizeof(g_error), fmt, ap);
	va_end(ap);
}
#define LTEN_M_CHECK(expr)                                                                                       \
	do {                                                                                                     \
		hipError_t e_ = (expr);                                                                          \
		if (e_ != hipSuccess) {                                                                          \
			set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);      \
			return 1;                                                                                \
		}                                                                                                \
	} while (0)
#define LTEN_M_REQUIRE(cond, ...)                                                                                \
	do {                                                                                                     \
		if (!(cond)) {                                                                                   \
			set_error(__VA_ARGS__);                                                                  \
			return 2;                                                                                \
		}                                                                                                \
	} while (0)

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_i8_peak_kernel(int iters, int* sink, long long* clocks)
{
	v16i acc0 = {}, acc1 = {}, acc2 = {}, acc3 = {};
	v4i a = { (int)threadIdx.x, 1, 2, 3 }, b = { 4, 5, (int)blockIdx.x, 7 };
	const long long c0 = clock64(), w0 = wall_clock64();
	for (int i = 0; i < iters; i++) {
		acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc0, 0, 0, 0);
		acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc1, 0, 0, 0);
		acc2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc2, 0, 0, 0);
		acc3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc3, 0, 0, 0);
	}
	int s = 0;
	for (int r = 0; r < 16; r++) s += acc0[r] + acc1[r] + acc2[r] + acc3[r];
	if (clocks && blockIdx.x == 0 && threadIdx.x == 0) {
		clocks[0] = clock64() - c0;       // shader clocks spent in the loop
		clocks[1] = wall_clock64() - w0;  // same span in the 100 MHz wall clock
	}
	if (s == 0x7fffffff) *sink = s;  // keeps the loop alive without a store in practice
}

__global__ __launch_bounds__(256) void mfma_f32_peak_kernel(int iters, float* sink)
{
	v16f acc0 = {}, acc1 = {}, acc2 = {}, acc3 = {};
	float a = (float)threadIdx.x, b = (float)blockIdx.x;
	for (int i = 0; i < iters; i++) {
		acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc0, 0, 0, 0);
		acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc1, 0, 0, 0);
		acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc2, 0, 0, 0);
		acc3 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc3, 0, 0, 0);
	}
	float s = 0;
	for (int r = 0; r < 16; r++) s += acc0[r] + acc1[r] + acc2[r] + acc3[r];
	if (s == 12345.678f) *sink = s;
}

// The same loops on operands that look like data: every lane holds eight pseudo-random register sets per operand and
// every MFMA takes another pair, so the multiplier inputs toggle as they do in a GEMM (with the constant operands
// above they do not, and the part draws much less power).
__device__ __forceinline__ unsigned mix32(unsigned x)
{
	x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
	return x;
}

__global__ __launch_bounds__(256) void mfma_i8_peak_random_kernel(int iters, int* sink, long long* clocks)
{
	v16i acc0 = {}, acc1 = {}, acc2 = {}, acc3 = {};
	v4i a[8], b[8];
	unsigned seed = (blockIdx.x * 256 + threadIdx.x) * 97u + 12345u;
#pragma unroll
	for (int i = 0; i < 8; i++) {
		a[i] = v4i{ (int)mix32(seed + 8 * i), (int)mix32(seed + 8 * i + 1), (int)mix32(seed + 8 * i + 2), (int)mix32(seed + 8 * i + 3) };
		b[i] = v4i{ (int)mix32(seed + 8 * i + 4), (int)mix32(seed + 8 * i + 5), (int)mix32(seed + 8 * i + 6), (int)mix32(seed + 8 * i + 7) };
	}
	const long long c0 = clock64(), w0 = wall_clock64();
	for (int i = 0; i < iters; i += 2) {
#pragma unroll
		for (int u = 0; u < 2; u++) {
			acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 0], b[4 * u + 0], acc0, 0, 0, 0);
			acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 1], b[4 * u + 1], acc1, 0, 0, 0);
			acc2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 2], b[4 * u + 2], acc2, 0, 0, 0);
			acc3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 3], b[4 * u + 3], acc3, 0, 0, 0);
		}
	}
	int s = 0;
	for (int r = 0; r < 16; r++) s += acc0[r] + acc1[r] + acc2[r] + acc3[r];
	if (clocks && blockIdx.x == 0 && threadIdx.x == 0) {
		clocks[0] = clock64() - c0;
		clocks[1] = wall_clock64() - w0;
	}
	if (s == 0x7fffffff) *sink = s;
}

__global__ __launch_bounds__(256) void mfma_f32_peak_random_kernel(int iters, float* sink)
{
	v16f acc0 = {}, acc1 = {}, acc2 = {}, acc3 = {};
	float a[8], b[8];
	unsigned seed = (blockIdx.x * 256 + threadIdx.x) * 97u + 12345u;
#pragma unroll
	for (int i = 0; i < 8; i++) {
		a[i] = (float)(int)(mix32(seed + 2 * i) >> 8) * (1.0f / 8388608.0f) - 1.0f;      // uniform in [-1, 1)
		b[i] = (float)(int)(mix32(seed + 2 * i + 1) >> 8) * (1.0f / 8388608.0f) - 1.0f;
	}
	for (int i = 0; i < iters; i += 2) {
#pragma unroll
		for (int u = 0; u < 2; u++) {
			acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * u + 0], b[4 * u + 0], acc0, 0, 0, 0);
			acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * u + 1], b[4 * u + 1], acc1, 0, 0, 0);
			acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * u + 2], b[4 * u + 2], acc2, 0, 0, 0);
			acc3 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * u + 3], b[4 * u + 3], acc3, 0, 0, 0);
		}
	}
	float s = 0;
	for (int r = 0; r < 16; r++) s += acc0[r] + acc1[r] + acc2[r] + acc3[r];
	if (s == 12345.678f) *sink = s;
}

__global__ __launch_bounds__(256) void copy_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, uint64_t n16)
{
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256) dst[i] = src[i];
}

// The int8 loop on operands taken from a caller's matrices: every lane loads eight 16-byte pieces of `a` and eight of
// `b` (at lane- and workgroup-dependent places, wrapping inside `bytes`), flips the sign bits of the `a` pieces as the
// GEMM does with l-ten's uint8 activations (`b` holds prepared int8 weights), and cycles through them: the multiplier
// inputs then have the value distribution of that product's operands, which is what the part's power draw depends on.
__global__ __launch_bounds__(256) void mfma_i8_peak_operands_kernel(int iters, const v4i* __restrict__ a_src, const v4i* __restrict__ b_src,
                                                                    unsigned n16, int* sink, long long* clocks)
{
	v16i acc0 = {}, acc1 = {}, acc2 = {}, acc3 = {};
	v4i a[8], b[8];
	const unsigned gid = blockIdx.x * 256 + threadIdx.x;
#pragma unroll
	for (int i = 0; i < 8; i++) {
		const unsigned at = (unsigned)(((uint64_t)gid * 8 + i) * 2654435761ull % n16);
		a[i] = a_src[at];
		a[i].x ^= 0x80808080; a[i].y ^= 0x80808080; a[i].z ^= 0x80808080; a[i].w ^= 0x80808080;
		b[i] = b_src[at];
	}
	const long long c0 = clock64(), w0 = wall_clock64();
	for (int i = 0; i < iters; i += 2) {
#pragma unroll
		for (int u = 0; u < 2; u++) {
			acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 0], b[4 * u + 0], acc0, 0, 0, 0);
			acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 1], b[4 * u + 1], acc1, 0, 0, 0);
			acc2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 2], b[4 * u + 2], acc2, 0, 0, 0);
			acc3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * u + 3], b[4 * u + 3], acc3, 0, 0, 0);
		}
	}
	int s = 0;
	for (int r = 0; r < 16; r++) s += acc0[r] + acc1[r] + acc2[r] + acc3[r];
	if (clocks && blockIdx.x == 0 && threadIdx.x == 0) {
		clocks[0] = clock64() - c0;
		clocks[1] = wall_clock64() - w0;
	}
	if (s == 0x7fffffff) *sink = s;
}

static double g_last_cycles_per_mfma = 0.0, g_last_shader_mhz = 0.0;

// kinds 0..3 as in the header; kind 4 = int8 on the caller's operands
static int run_peak(int kind, int waves_per_simd, const void* a, const void* b, uint64_t bytes, float* tera_per_s)
{
	hipDeviceProp_t prop;
	int dev = 0;
	LTEN_M_CHECK(hipGetDevice(&dev));
	LTEN_M_CHECK(hipGetDeviceProperties(&prop, dev));
	const int blocks = prop.multiProcessorCount * waves_per_simd;  // 4 waves per block = 1 per SIMD
	const bool int8 = kind == 0 || kind == 2 || kind == 4;
	const int iters = int8 ? 4096 : 2048;
	void* sink = nullptr;
	LTEN_M_CHECK(hipMalloc(&sink, 64));
	hipEvent_t e0, e1;
	LTEN_M_CHECK(hipEventCreate(&e0));
	LTEN_M_CHECK(hipEventCreate(&e1));
	float best = 1e30f;
	for (int rep = 0; rep < 4; rep++) {
		LTEN_M_CHECK(hipEventRecord(e0, nullptr));
		if (kind == 0)
			mfma_i8_peak_kernel<<<dim3(blocks), dim3(256)>>>(iters, static_cast<int*>(sink), static_cast<long long*>(sink) + 1);
		else if (kind == 2)
			mfma_i8_peak_random_kernel<<<dim3(blocks), dim3(256)>>>(iters, static_cast<int*>(sink), static_cast<long long*>(sink) + 1);
		else if (kind == 4)
			mfma_i8_peak_operands_kernel<<<dim3(blocks), dim3(256)>>>(iters, static_cast<const v4i*>(a), static_cast<const v4i*>(b), (unsigned)(bytes / 16),
			                                                          static_cast<int*>(sink), static_cast<long long*>(sink) + 1);
		else if (kind == 1)
			mfma_f32_peak_kernel<<<dim3(blocks), dim3(256)>>>(iters, static_cast<float*>(sink));
		else
			mfma_f32_peak_random_kernel<<<dim3(blocks), dim3(256)>>>(iters, static_cast<float*>(sink));
		LTEN_M_CHECK(hipGetLastError());
		LTEN_M_CHECK(hipEventRecord(e1, nullptr));
		LTEN_M_CHECK(hipEventSynchronize(e1));
		float ms = 0;
		LTEN_M_CHECK(hipEventElapsedTime(&ms, e0, e1));
		if (rep > 0 && ms < best) best = ms;
	}
	const double ops_per_mfma = int8 ? 2.0 * 32 * 32 * 32 : 2.0 * 32 * 32 * 2;
	*tera_per_s = (float)(ops_per_mfma * 4.0 * iters * 4.0 * blocks / (best * 1e-3) / 1e12);
	if (int8) {
		long long clk[2] = { 0, 0 };
		LTEN_M_CHECK(hipMemcpy(clk, static_cast<long long*>(sink) + 1, sizeof(clk), hipMemcpyDeviceToHost));
		g_last_cycles_per_mfma = (double)clk[0] / (4.0 * iters);
		g_last_shader_mhz = clk[1] > 0 ? (double)clk[0] / ((double)clk[1] / 100.0) : 0.0;
	}
	hipEventDestroy(e0);
	hipEventDestroy(e1);
	LTEN_M_CHECK(hipFree(sink));
	return 0;
}

}  // namespace lten_measure

using namespace lten_measure;

extern "C" {

const char* lten_measure_last_error(void) { return g_error; }

int lten_measure_mfma_peak(int kind, int waves_per_simd, float* tera_per_s)
{
	LTEN_M_REQUIRE(tera_per_s != nullptr && kind >= 0 && kind <= 3 && waves_per_simd >= 1 && waves_per_simd <= 8, "lten_measure_mfma_peak: bad argument");
	return run_peak(kind, waves_per_simd, nullptr, nullptr, 0, tera_per_s);
}

int lten_measure_mfma_peak_operands(const void* a_u8, const void* b_i8, uint64_t bytes, int waves_per_simd, float* tera_per_s)
{
	LTEN_M_REQUIRE(tera_per_s != nullptr && a_u8 != nullptr && b_i8 != nullptr && bytes >= 4096 && bytes < (1ull << 35) && waves_per_simd >= 1 &&
	                   waves_per_simd <= 8 && ((reinterpret_cast<uintptr_t>(a_u8) | reinterpret_cast<uintptr_t>(b_i8)) & 15) == 0,
	               "lten_measure_mfma_peak_operands: bad argument");
	return run_peak(4, waves_per_simd, a_u8, b_i8, bytes, tera_per_s);
}

int lten_measure_last_clocks(double* cycles_per_mfma, double* shader_mhz)
{
	if (cycles_per_mfma) *cycles_per_mfma = g_last_cycles_per_mfma;
	if (shader_mhz) *shader_mhz = g_last_shader_mhz;
	return 0;
}

int lten_measure_copy(const void* src, void* dst, uint64_t bytes)
{
	LTEN_M_REQUIRE((bytes & 15) == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0,
	               "lten_measure_copy: size and pointers must be multiples of 16");
	if (bytes == 0) return 0;
	const uint64_t n16 = bytes / 16;
	const unsigned blocks = (unsigned)std::min<uint64_t>((n16 + 255) / 256, 256 * 32);
	copy_kernel<<<dim3(blocks), dim3(256)>>>(static_cast<const v4i*>(src), static_cast<v4i*>(dst), n16);
	LTEN_M_CHECK(hipGetLastError());
	return 0;
}

}  // extern "C"
