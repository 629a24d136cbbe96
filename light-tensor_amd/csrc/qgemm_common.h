// Definitions shared by the int8 GEMM kernels: the problem descriptor handed to every kernel, the LDS
// chunk swizzle and the requantize step.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

namespace lten_hip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

enum QOut { Q_OUT_U8_FAST = 0, Q_OUT_U8_EXACT = 1, Q_OUT_ACC = 2 };

struct QProblem {
	const uint8_t* A;  // element (m, k) at A[m * a_rs + k * a_ks]
	const uint8_t* B;  // element (n, k) at B[n * b_rs + k * b_ks]
	void* C;           // uint8 [M x N] or int32 [M x N], row-major, ld = N
	int64_t a_rs, a_ks, b_rs, b_ks;
	int M, N, K;
	// Rows padded to a multiple of 16 bytes: the last k_pad of the K bytes of every row of A and B are padding that holds
	// the byte 128 (0 in a prepared B), which multiplies to nothing; konst already allows for what the padding adds to
	// byte sums taken over all K bytes of a row, and kernels that need the number of real bytes use K - k_pad
	int k_pad = 0;
	const int32_t* rterm;  // [M] (128 - zpB) * SA_m, or null
	const int32_t* cterm;  // [N] (128 - zpA) * SB_n + bias_n, or null
	int32_t konst;         // K (zpA zpB - 16384) over the real bytes, less what padding bytes add to the two sum terms
	float mult;            // real_multiplier
	float zp_c;            // (float) output zero point
	int vec_ok;            // operand bases and row strides are multiples of 16 bytes
	// 0x80808080 when B holds l-ten's uint8 bytes (XORed into int8 on the way into the MFMA), 0 when B was prepared
	// by lten_hip_fcq_prepare_weights and already holds the int8 values b - 128
	uint32_t b_flip;
	// split-K launches of the direct-to-LDS tiles: `splits` workgroups share an output tile, each takes K / splits
	int32_t* split_partial;     // [tile][split][T*T] partial sums in register order
	unsigned* split_counters;   // [tile] arrivals; zero between launches
	int splits;
	// Zero-point terms worked out by the tiled kernel itself (prepared weights only; rterm and cterm are null then):
	// the column term is coef_b * wsum[n] + bias[n] with wsum the weight rows' byte sums kept since the weights were
	// prepared, the row term coef_a * (byte sum of activation row m), which the kernel takes from the operand
	// fragments it feeds to the matrix cores.  l-ten/math_fns.cpp:1362-1380 computes both on every call.
	const int32_t* wsum = nullptr;  // [N] sum_k W[n][k] of the uint8 weight bytes, 16-byte aligned; null = not fused
	const int32_t* bias = nullptr;  // [N] or null (fused form only)
	int coef_a = 0;                 // 128 - zpB
	int coef_b = 0;                 // 128 - zpA
	int32_t acc_offset = 0;         // set by the tiled kernels' launchers: see accumulator_offset (qgemm_fast.hip)
};

// 16-byte-chunk swizzle: chunk kc of tile row `row` lives at chunk kc ^ swz(row).
// Chosen so that any aligned group of 8 or of 16 consecutive rows, read at one logical
// chunk, touches every LDS bank group once (both for 32 and for 64 four-byte banks).
template <int CPR>
__device__ __forceinline__ int swz(int row)
{
	if (CPR == 2) return ((row >> 2) ^ (row >> 3)) & 1;
	if (CPR == 4) return ((row >> 2) & 1) | ((((row >> 1) ^ (row >> 3)) & 1) << 1);
	if (CPR == 8) return ((row ^ (row >> 3)) & 1) | (row & 6);
	return 0;
}

__device__ __forceinline__ v4i flip_sign_bits(v4i v)
{
	v.x ^= 0x80808080;
	v.y ^= 0x80808080;
	v.z ^= 0x80808080;
	v.w ^= 0x80808080;
	return v;
}

// The same with a wave-uniform pattern: QProblem::b_flip for the weight operand.
__device__ __forceinline__ v4i flip_bits(v4i v, uint32_t pattern)
{
	v.x ^= (int)pattern;
	v.y ^= (int)pattern;
	v.z ^= (int)pattern;
	v.w ^= (int)pattern;
	return v;
}

// requant<Q_OUT_U8_FAST> whose result byte lands in byte BYTE of `word`, the other bytes untouched: the
// convert instruction writes its low byte there itself, so packing four outputs costs no further instruction.
template <int BYTE>
__device__ __forceinline__ void requant_into(unsigned& word, int acc, float mult, float zp)
{
#pragma clang fp contract(off)
	float prod = (float)acc * mult;
	float s = prod + zp;
	if (BYTE == 0) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(word) : "v"(s));
	if (BYTE == 1) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(word) : "v"(s));
	if (BYTE == 2) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(word) : "v"(s));
	if (BYTE == 3) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(word) : "v"(s));
}

// Exact image of l-ten/math_fns.cpp:1474 for one accumulator.
template <int OUT>
__device__ __forceinline__ unsigned requant(int acc, float mult, float zp)
{
	// Two separately rounded operations: a fused multiply-add rounds once and differs in the last bit.
#pragma clang fp contract(off)
	float prod = (float)acc * mult;
	float s = prod + zp;
	if (OUT == Q_OUT_U8_EXACT) {
		// x86 cvttss2si: NaN and anything outside [-2^31, 2^31) give 0x80000000.
		int i = (s >= -2147483648.0f && s < 2147483648.0f) ? (int)s : (int)0x80000000;
		return (unsigned)i & 0xFFu;
	}
	return (unsigned)(int)s & 0xFFu;  // caller guarantees |s| < 2^31
}


// Weight-streaming kernel for M <= 16 (qskinny.hip); computes its own zero-point sums.  -1 = does not fit.
int qskinny_dispatch(const QProblem& p, int out, const int32_t* bias, int zp_a, int zp_b);

// One-launch kernel for small NT products (qdirect.hip); computes its own zero-point sums.  -1 = does not fit.
int qdirect_dispatch(const QProblem& p, int out, const int32_t* bias, int zp_a, int zp_b);

// Dispatch of the tuned square-ish kernels (qgemm_fast.hip).  Returns -1 when no fast variant fits.
int qgemm_fast_dispatch(const QProblem& p, int out, int variant);
// Split-K launch; scratch == nullptr takes the library's own buffers (allocated on first use), otherwise the
// caller's SplitScratch (the entry point that allocates nothing hands in its static device array).
struct SplitScratch {
	int32_t* partial;
	size_t partial_bytes;
	unsigned* counters;  // zero between launches
	int max_tiles;
};
int qgemm_fast_split_dispatch(const QProblem& p, int out, int splits, const SplitScratch* scratch);

}  // namespace lten_hip
