// Weight-streaming int8 FC for skinny activations (M <= 16 rows against W[N x K], both contiguous in K).
//
// The work is one pass over W (N*K bytes, read once from HBM); everything else is noise, so the kernel is
// organised around that stream.  A workgroup owns 16 consecutive rows of W; its 8 wavefronts split K among
// themselves.  Each wavefront pulls its [16 rows x K/8] slab into LDS with direct global->LDS loads — one
// wave-wide load covers 1 KB of one row, so every request is a run of whole cache lines — keeps the whole
// slab in flight at once (128 KB per CU), then walks it with ds_read_b128 in the lane layout of the
// 16x16x64 int8 MFMA (lane -> row lane%16, 16-byte k-group lane/16).  Rows are padded by 16 bytes in LDS
// so that the 16 rows a read touches fall in different banks.  The activations (at most 16 x K bytes,
// L2 resident) are fetched straight into the other MFMA operand; rows beyond M read as the zero of the
// signed domain.  The 8 partial 16x16 accumulators meet in LDS, and one wavefront applies the zero-point
// terms and the requantize of l-ten/math_fns.cpp:1469-1474 and writes the M x 16 outputs.
//
// As in the tiled kernels, bytes are XORed with 0x80 on their way into the MFMA (uint8 -> int8) and the
// identity in qgemm.hip restores l-ten's accumulator; the byte sums it needs are taken from the same
// registers with dot4 instructions, only when their coefficient is non-zero.
#include "common.h"
#include "qgemm_common.h"

namespace lten_hip {

__device__ __forceinline__ void skinny_async_load16(uint32_t lds_addr, const uint8_t* base, uint32_t voff)
{
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

template <int WAVES, int KW, int OUT, bool SUM_A, bool SUM_B>
__global__ __launch_bounds__(WAVES * 64) void qskinny_kernel(QProblem p, const int32_t* bias, int coef_a, int coef_b)
{
	// KW = bytes of K per wavefront (multiple of 1024): K == WAVES * KW
	constexpr int ROW = KW + 16;         // padded LDS row pitch
	constexpr int SLAB = 16 * ROW;       // one wavefront's slab
	constexpr int LOADS_PER_ROW = KW / 1024;
	__shared__ __attribute__((aligned(1024))) uint8_t smem[WAVES * SLAB > WAVES * 1024 ? WAVES * SLAB : WAVES * 1024];
	__shared__ int sums_a[WAVES][16], sums_b[WAVES][16];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int n0 = blockIdx.x * 16;
	const int kbeg = wave * KW;
	const uint32_t slab_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem + wave * SLAB;

	// the whole slab goes in flight before anything is consumed
#pragma unroll
	for (int r = 0; r < 16; r++)
#pragma unroll
		for (int c = 0; c < LOADS_PER_ROW; c++)
			skinny_async_load16(slab_addr + r * ROW + c * 1024, p.B + (int64_t)(n0 + r) * p.K + kbeg + c * 1024, lane * 16);

	const int lrow = lane & 15, lgrp = lane >> 4;
	const uint8_t* xrow = p.A + (int64_t)lrow * p.K + kbeg + lgrp * 16;
	const bool xvalid = lrow < p.M;
	const uint8_t* wfrag = smem + wave * SLAB + lrow * ROW + lgrp * 16;

	v4i acc = { 0, 0, 0, 0 };
	int sa = 0, sb = 0;
	constexpr int STEPS = KW / 64;
	v4i fx[STEPS];
#pragma unroll
	for (int s = 0; s < STEPS; s++) {
		fx[s] = v4i{ (int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080 };
		if (xvalid) fx[s] = *reinterpret_cast<const v4i*>(xrow + s * 64);
	}
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // own slab and activations have landed (no other wave reads this slab)
#pragma unroll
	for (int s = 0; s < STEPS; s++) {
		v4i fw = *reinterpret_cast<const v4i*>(wfrag + s * 64);
		fw = flip_sign_bits(fw);
		const v4i fa = flip_sign_bits(fx[s]);
		if (SUM_B) {
			sb = __builtin_amdgcn_sdot4(fw.x, 0x01010101, sb, false);
			sb = __builtin_amdgcn_sdot4(fw.y, 0x01010101, sb, false);
			sb = __builtin_amdgcn_sdot4(fw.z, 0x01010101, sb, false);
			sb = __builtin_amdgcn_sdot4(fw.w, 0x01010101, sb, false);
		}
		if (SUM_A) {
			sa = __builtin_amdgcn_sdot4(fa.x, 0x01010101, sa, false);
			sa = __builtin_amdgcn_sdot4(fa.y, 0x01010101, sa, false);
			sa = __builtin_amdgcn_sdot4(fa.z, 0x01010101, sa, false);
			sa = __builtin_amdgcn_sdot4(fa.w, 0x01010101, sa, false);
		}
		// MFMA A operand = activations (rows m), B operand = weights (columns n):
		// lane (lrow, lgrp), register e holds out[m = 4*lgrp + e][n = lrow]
		acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa, fw, acc, 0, 0, 0);
	}
	if (SUM_A || SUM_B) {
		// a lane holds the sums of its 16-byte k-group only: fold the four k-groups (lanes l, l+16, l+32, l+48)
		sa += __shfl_xor(sa, 16, 64); sa += __shfl_xor(sa, 32, 64);
		sb += __shfl_xor(sb, 16, 64); sb += __shfl_xor(sb, 32, 64);
		if (lane < 16) { sums_a[wave][lane] = sa; sums_b[wave][lane] = sb; }
	}

	// partial accumulators of the 8 k-slices meet in LDS (each wave overwrites the head of its own slab)
	__syncthreads();
	*reinterpret_cast<v4i*>(smem + wave * 1024 + lane * 16) = acc;
	__syncthreads();
	if (wave != 0) return;
	v4i tot = { 0, 0, 0, 0 };
#pragma unroll
	for (int w = 0; w < WAVES; w++) tot += *reinterpret_cast<const v4i*>(smem + w * 1024 + lane * 16);
	int tsa[4] = { 0, 0, 0, 0 }, tsb = 0;
	if (SUM_A || SUM_B) {
#pragma unroll
		for (int w = 0; w < WAVES; w++) {
			tsb += sums_b[w][lrow];
#pragma unroll
			for (int e = 0; e < 4; e++) tsa[e] += sums_a[w][lgrp * 4 + e];
		}
	}
	const int n = n0 + lrow;
	// sum a'b' -> l-ten's element: + coef_a * sum_k a' + coef_b * sum_k b' + K * coef_a * coef_b (+ bias)
	//   with a' = a - 128, coef_a = 128 - zpB, coef_b = 128 - zpA
	const int base = coef_b * tsb + p.K * coef_a * coef_b + (bias ? bias[n] : 0);
#pragma unroll
	for (int e = 0; e < 4; e++) {
		const int m = lgrp * 4 + e;
		if (m >= p.M) continue;
		const int v = tot[e] + base + coef_a * tsa[e];
		if (OUT == Q_OUT_ACC) static_cast<int*>(p.C)[(int64_t)m * p.N + n] = v;
		else static_cast<uint8_t*>(p.C)[(int64_t)m * p.N + n] = (uint8_t)requant<OUT>(v, p.mult, p.zp_c);
	}
}

template <int WAVES, int KW>
static int launch_skinny(const QProblem& p, int out, const int32_t* bias, int coef_a, int coef_b, const char* name)
{
	const dim3 grid((unsigned)(p.N / 16)), block(WAVES * 64);
	set_kernel_name(name);
	const bool sum_a = coef_a != 0, sum_b = coef_b != 0;
#define LTEN_SK(OUTV, SA, SB) qskinny_kernel<WAVES, KW, OUTV, SA, SB><<<grid, block, 0, stream()>>>(p, bias, coef_a, coef_b)
#define LTEN_SK_OUT(OUTV)                                     \
	if (sum_a && sum_b) LTEN_SK(OUTV, true, true);        \
	else if (sum_a) LTEN_SK(OUTV, true, false);           \
	else if (sum_b) LTEN_SK(OUTV, false, true);           \
	else LTEN_SK(OUTV, false, false);
	if (out == Q_OUT_U8_FAST) { LTEN_SK_OUT(Q_OUT_U8_FAST) }
	else if (out == Q_OUT_U8_EXACT) { LTEN_SK_OUT(Q_OUT_U8_EXACT) }
	else { LTEN_SK_OUT(Q_OUT_ACC) }
#undef LTEN_SK_OUT
#undef LTEN_SK
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// Returns -1 when the problem does not fit the streaming kernel (the caller then uses the tiled kernels).
int qskinny_dispatch(const QProblem& p, int out, const int32_t* bias, int zp_a, int zp_b)
{
	if (!(p.a_ks == 1 && p.b_ks == 1 && p.vec_ok && p.M >= 1 && p.M <= 16 && p.N % 16 == 0)) return -1;
	const int coef_a = 128 - zp_b, coef_b = 128 - zp_a;
	if (p.K == 8 * 1024) return launch_skinny<8, 1024>(p, out, bias, coef_a, coef_b, "qskinny_mfma_w8_k1024");
	if (p.K == 4 * 1024) return launch_skinny<4, 1024>(p, out, bias, coef_a, coef_b, "qskinny_mfma_w4_k1024");
	if (p.K == 2 * 1024) return launch_skinny<2, 1024>(p, out, bias, coef_a, coef_b, "qskinny_mfma_w2_k1024");
	return -1;
}

}  // namespace lten_hip
