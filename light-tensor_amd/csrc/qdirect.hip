// int8 FC for small outputs (a few hundred 16x16 tiles): one launch, operands straight from global memory.
//
// At these sizes (e.g. l-ten's 64 x 784 MNIST batch against a 512 x 784 weight matrix) the run time is launch
// and memory latency, not arithmetic, so the kernel is one dependent chain as short as possible: a workgroup
// owns one 16 x 16 output tile, its wavefronts split K in 64-byte steps (wavefront w takes steps w, w + WAVES,
// ...), every lane loads the 16 bytes the 16x16x64 int8 MFMA wants from it (row lane % 16, k-group lane / 16)
// for all its steps at once, and the zero-point byte sums come from the same registers with dot4 instructions
// — no separate row-sum launch.  The partial tiles and sums meet in LDS and wavefront 0 applies the identity
// of qgemm.hip and the requantize of l-ten/math_fns.cpp:1469-1474.
//
// K only has to be a multiple of 16 (k-groups past K read as the zero of the signed domain).
#include "common.h"
#include "qgemm_common.h"

namespace lten_hip {

template <int WAVES, int OUT>
__global__ __launch_bounds__(WAVES * 64) void qdirect_kernel(QProblem p, const int32_t* bias, int coef_a, int coef_b)
{
	constexpr int U = 4;  // steps in flight per wavefront and pass
	__shared__ __attribute__((aligned(16))) int partial[WAVES][64 * 4];
	__shared__ int sums_a[WAVES][16], sums_b[WAVES][16];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int lrow = lane & 15, lgrp = lane >> 4;
	const int tiles_n = (p.N + 15) / 16;
	const int m0 = (blockIdx.x / tiles_n) * 16, n0 = (blockIdx.x % tiles_n) * 16;
	const bool a_ok = m0 + lrow < p.M, b_ok = n0 + lrow < p.N;
	const uint8_t* arow = p.A + (int64_t)(m0 + lrow) * p.a_rs + lgrp * 16;
	const uint8_t* brow = p.B + (int64_t)(n0 + lrow) * p.b_rs + lgrp * 16;
	const int steps = (p.K + 63) / 64;
	const v4i zero = { (int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080 };
	const v4i zero_b = { (int)p.b_flip, (int)p.b_flip, (int)p.b_flip, (int)p.b_flip };  // prepared weights: int8 zeros

	v4i acc = { 0, 0, 0, 0 };
	int sa = 0, sb = 0;
	for (int s0 = wave; s0 < steps; s0 += WAVES * U) {
		v4i fa[U], fb[U];
#pragma unroll
		for (int u = 0; u < U; u++) {
			const int k = (s0 + u * WAVES) * 64 + lgrp * 16;
			fa[u] = zero;
			fb[u] = zero_b;
			if (k < p.K) {
				if (a_ok) fa[u] = *reinterpret_cast<const v4i*>(arow + (int64_t)(s0 + u * WAVES) * 64);
				if (b_ok) fb[u] = *reinterpret_cast<const v4i*>(brow + (int64_t)(s0 + u * WAVES) * 64);
			}
		}
#pragma unroll
		for (int u = 0; u < U; u++) {
			const v4i a = flip_sign_bits(fa[u]), b = flip_bits(fb[u], p.b_flip);
			sa = __builtin_amdgcn_sdot4(a.x, 0x01010101, sa, false);
			sa = __builtin_amdgcn_sdot4(a.y, 0x01010101, sa, false);
			sa = __builtin_amdgcn_sdot4(a.z, 0x01010101, sa, false);
			sa = __builtin_amdgcn_sdot4(a.w, 0x01010101, sa, false);
			sb = __builtin_amdgcn_sdot4(b.x, 0x01010101, sb, false);
			sb = __builtin_amdgcn_sdot4(b.y, 0x01010101, sb, false);
			sb = __builtin_amdgcn_sdot4(b.z, 0x01010101, sb, false);
			sb = __builtin_amdgcn_sdot4(b.w, 0x01010101, sb, false);
			// lane (lrow, lgrp), register e holds out[m = 4*lgrp + e][n = lrow]
			acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc, 0, 0, 0);
		}
	}
	// a lane holds the byte sums of its 16-byte k-groups only: fold the four k-groups (lanes l, l+16, l+32, l+48)
	sa += __shfl_xor(sa, 16, 64); sa += __shfl_xor(sa, 32, 64);
	sb += __shfl_xor(sb, 16, 64); sb += __shfl_xor(sb, 32, 64);
	if (lane < 16) { sums_a[wave][lane] = sa; sums_b[wave][lane] = sb; }
	*reinterpret_cast<v4i*>(&partial[wave][lane * 4]) = acc;
	__syncthreads();
	if (wave != 0) return;

	v4i tot = { 0, 0, 0, 0 };
	int tsa[4] = { 0, 0, 0, 0 }, tsb = 0;
#pragma unroll
	for (int w = 0; w < WAVES; w++) {
		tot += *reinterpret_cast<const v4i*>(&partial[w][lane * 4]);
		tsb += sums_b[w][lrow];
#pragma unroll
		for (int e = 0; e < 4; e++) tsa[e] += sums_a[w][lgrp * 4 + e];
	}
	const int n = n0 + lrow;
	if (n >= p.N) return;
	// sum a'b' -> l-ten's element: + coef_a * sum_k a' + coef_b * sum_k b' + K * coef_a * coef_b (+ bias)
	//   with a' = a - 128, coef_a = 128 - zpB, coef_b = 128 - zpA
	const int base = coef_b * tsb + (p.K - p.k_pad) * coef_a * coef_b + (bias ? bias[n] : 0);
#pragma unroll
	for (int e = 0; e < 4; e++) {
		const int m = m0 + lgrp * 4 + e;
		if (m >= p.M) continue;
		const int v = tot[e] + base + coef_a * tsa[e];
		if (OUT == Q_OUT_ACC) static_cast<int*>(p.C)[(int64_t)m * p.N + n] = v;
		else static_cast<uint8_t*>(p.C)[(int64_t)m * p.N + n] = (uint8_t)requant<OUT>(v, p.mult, p.zp_c);
	}
}

// Returns -1 when the problem is not a small NT product with 16-byte aligned rows.
int qdirect_dispatch(const QProblem& p, int out, const int32_t* bias, int zp_a, int zp_b)
{
	if (!(p.a_ks == 1 && p.b_ks == 1 && p.vec_ok && p.K % 16 == 0 && p.M >= 1 && p.N >= 1 && p.K >= 1)) return -1;
	const int64_t tiles = (int64_t)ceil_div((uint64_t)p.M, 16) * ceil_div((uint64_t)p.N, 16);
	// Up to 8192 tiles, as long as this kernel is ahead of the 128 x 128 direct-to-LDS tiles where those apply (at least
	// 64 output columns, K >= 512 or at least 64 such tiles: qgemm_dispatch).  It takes about 2.3 us + 4.1 us per million
	// (tiles x K), they about 5.4 us + 0.33 us per k-step of 128 bytes of a workgroup's share of K while they run in one
	// round, 4 us more when workgroups share tiles (split K, as qgemm_dispatch picks it), 2 us more when N is no multiple
	// of 4 (rows of the output that start on any byte), 2.5 us more with a partial last k-step.  300 x 1000 x 512: 4.8 us here, 6.9 there; 400 x 400 x 2048: 7.7
	// and 10.8; 256 x 512 x 4096: 9.4 and 13.8; 200 x 2000 x 256: 4.3 (13.8 on the guarded kernel, which took it before);
	// 1024 x 1000 x 1024: 16.8 and 8.6; 128 x 4096 x 1024: 9.6 and 7.4; 128 x 1024 x 16384: 30.3 and 23.3.  A few output
	// columns make poor use of 128-column tiles and stay here (4096 x 50 x 5760, l-ten's quantized MNIST layer at a large
	// batch: 22.5 us).
	if (tiles > 8192 || p.K > 16384) return -1;
	const uint64_t tiles128 = ceil_div((uint64_t)p.M, 128) * ceil_div((uint64_t)p.N, 128);
	// (from 64 output columns on: half-empty 128-column tiles still beat this kernel on long or many rows, 4096 x 100 x 9216 58 -> 25
	// us, 16384 x 64 x 1024 17 -> 7.5 us; at 50 columns, l-ten's layer above, they are level)
	const bool tiles_apply = p.N >= 64 && (p.K >= 512 || (p.K >= 32 && tiles128 >= 64)) && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0 &&
	                         (uint64_t)p.M * p.K < (1ull << 32) && (uint64_t)p.N * p.K < (1ull << 32);
	if (tiles_apply) {
		const int splits = (tiles128 <= 64 && p.K >= 8192) ? (tiles128 <= 32 ? 4 : 2) : (tiles128 <= 32 && p.K >= 4096) ? 2 : 1;
		const double here = 2.3 + 4.1e-6 * (double)tiles * p.K;
		const double there = 5.4 + 0.0026 * p.K / splits + (splits > 1 ? 4.0 : 0.0) + (p.N % 4 != 0 ? 2.0 : 0.0) + (p.K % 128 != 0 ? 2.5 : 0.0);
		if (here >= there) return -1;
	}
	const int coef_a = 128 - zp_b, coef_b = 128 - zp_a;
	const dim3 grid((unsigned)tiles);
	if (p.K <= 1024) {
		set_kernel_name("qdirect_16x16_w4");
		if (out == Q_OUT_U8_FAST) qdirect_kernel<4, Q_OUT_U8_FAST><<<grid, dim3(256), 0, stream()>>>(p, bias, coef_a, coef_b);
		else if (out == Q_OUT_U8_EXACT) qdirect_kernel<4, Q_OUT_U8_EXACT><<<grid, dim3(256), 0, stream()>>>(p, bias, coef_a, coef_b);
		else qdirect_kernel<4, Q_OUT_ACC><<<grid, dim3(256), 0, stream()>>>(p, bias, coef_a, coef_b);
	} else {
		set_kernel_name("qdirect_16x16_w8");
		if (out == Q_OUT_U8_FAST) qdirect_kernel<8, Q_OUT_U8_FAST><<<grid, dim3(512), 0, stream()>>>(p, bias, coef_a, coef_b);
		else if (out == Q_OUT_U8_EXACT) qdirect_kernel<8, Q_OUT_U8_EXACT><<<grid, dim3(512), 0, stream()>>>(p, bias, coef_a, coef_b);
		else qdirect_kernel<8, Q_OUT_ACC><<<grid, dim3(512), 0, stream()>>>(p, bias, coef_a, coef_b);
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
