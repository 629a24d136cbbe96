// Weight-streaming int8 FC for skinny activations (M <= 32 rows against W[N x K], both contiguous in K, K any multiple
// of 16 up to 8192 — up to 16384 for M <= 16, beyond that in chunks of K with a launch that adds them — and any N).
//
// The work is one pass over W (N*K bytes, read once from HBM); everything else is noise, so the kernel is
// organised around that stream.  A workgroup takes 16 consecutive rows of W at a time (then the next such
// group, one workgroup per CU); its 8 wavefronts split K among themselves.  Each wavefront pulls its [16 rows x K/8] slab into LDS with direct global->LDS loads — one
// wave-wide load covers 1 KB of one row, so every request is a run of whole cache lines — keeps the whole
// slab in flight at once (128 KB per CU), then walks it with ds_read_b128 in the lane layout of the
// 16x16x64 int8 MFMA (lane -> row lane%16, 16-byte k-group lane/16).  Rows are padded by 16 bytes in LDS
// so that the 16 rows a read touches fall in different banks.  The activations (at most 16 x K bytes,
// L2 resident) are fetched straight into the other MFMA operand once per workgroup and stay in registers
// for all its row groups; rows beyond M read as the zero of the signed domain.  The 8 partial 16x16 accumulators meet in LDS, and one wavefront applies the zero-point
// terms and the requantize of l-ten/math_fns.cpp:1469-1474 and writes the M x 16 outputs.
//
// As in the tiled kernels, bytes are XORed with 0x80 on their way into the MFMA (uint8 -> int8) and the
// identity in qgemm.hip restores l-ten's accumulator; the byte sums it needs are taken from the same
// registers with dot4 instructions, only when their coefficient is non-zero.
#include "common.h"
#include "qgemm_common.h"
#include "lds_async.h"

#include <algorithm>

namespace lten_hip {

template <int WAVES, int SMAX, int MB, int OUT, bool SUM_A, bool SUM_B, bool CHUNKS = false>
__global__ __launch_bounds__(WAVES * 64) void qskinny_kernel(QProblem p, const int32_t* bias, int coef_a, int coef_b, int kw, int chunk_k)
{
	// CHUNKS (int32 sums only): K in chunks over blockIdx.y, chunk y takes k from y * chunk_k on and writes its sums to the
	// y-th [M x N] matrix behind C; the bias goes with the first chunk, the padding bytes are in the last
	const int k0 = CHUNKS ? (int)blockIdx.y * chunk_k : 0;
	const int Kc = CHUNKS ? min(chunk_k, p.K - k0) : p.K;
	const int pad_here = (!CHUNKS || k0 + chunk_k >= p.K) ? p.k_pad : 0;
	if (CHUNKS) {
		p.A += k0;
		p.B += k0;
		p.C = static_cast<int*>(p.C) + (int64_t)blockIdx.y * p.M * p.N;
		if (k0 != 0) bias = nullptr;
	}
	// kw = bytes of K per wavefront, a multiple of 64, at most SMAX * 64; wavefront w owns k in [w * kw, w * kw + kw) as
	// far as it lies inside K (any multiple of 16).  A slab holds 1 KB of 16 weight rows: SMAX / 16 passes per row group.
	constexpr int ROW = 1024 + 16;       // padded LDS row pitch
	constexpr int SLAB = 16 * ROW;       // one wavefront's slab
	constexpr int PASSES = SMAX / 16;
	__shared__ __attribute__((aligned(1024))) uint8_t smem[WAVES * SLAB];
	// PAR = 2: wave 0 reads one row group's partial tiles while the others already write the next group's (no second
	// barrier); with two row blocks only one copy fits beside the slabs, and a barrier ends every row group instead
	constexpr int PAR = MB == 1 ? 2 : 1;
	__shared__ __attribute__((aligned(16))) int partial[PAR][WAVES][MB][64 * 4];
	__shared__ int sums_a[WAVES][MB][16], sums_b[PAR][WAVES][16];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int kbeg = wave * kw;
	const int klen = max(0, min(kw, Kc - kbeg));    // this wavefront's share of K (0 for wavefronts past a short K)
	const int steps = (klen + 63) / 64;              // MFMA steps of 64 k; the last may be partial (K % 64 != 0)
	const uint32_t slab_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem + wave * SLAB;
	const int groups = (p.N + 15) / 16;

	// One pass of a row group's slab: 1 KB of each of the 16 rows, one wave-wide load per row (every request a run of whole
	// cache lines); lanes whose 16 bytes lie past the wavefront's share load nothing.  Rows past N repeat the last row;
	// their outputs are not stored.
	auto issue_slab = [&](int group, int pass) {
		// which lanes take part, as an execution mask: the addresses stay wave-uniform scalars outside any branch
		const uint64_t live = __ballot(pass * 1024 + lane * 16 < klen);
		if (live == 0) return;
#pragma unroll
		for (int r = 0; r < 16; r++) {
			const int row = min(group * 16 + r, p.N - 1);
			async_load16_masked_nt(live, slab_addr + r * ROW, p.B + (int64_t)row * p.K + kbeg + pass * 1024, lane * 16);
		}
	};
	// the activations of this wavefront's k-slice stay in registers for every row group the workgroup takes
	const int lrow = lane & 15, lgrp = lane >> 4;
	const uint8_t* wfrag = smem + wave * SLAB + lrow * ROW + lgrp * 16;
	v4i fx[MB][SMAX];  // activation rows mb * 16 + lrow
	int sa[MB];
	const v4i zero_u8 = { (int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080 };
	// They are fetched with four neighbouring lanes on the 64 bytes a row contributes to a step (lane 4 r + g: row r,
	// 16-byte group g), which the memory pipeline handles as one access per row, and exchanged into the MFMA layout
	// (lane r + 16 g) afterwards: fetched in the MFMA layout directly, neighbouring lanes name different rows and every
	// lane costs a cache look-up of its own (four times as many for 16 rows; 3 us of a 15 us kernel).
	// With fewer than four rows the exchange costs more than it saves and the lanes fetch in the MFMA layout.
	const bool exchange = p.M >= 4;
	const int ld_row = exchange ? lane >> 2 : lrow, ld_grp = exchange ? lane & 3 : lgrp;
#pragma unroll
	for (int mb = 0; mb < MB; mb++) {
		const uint8_t* xrow = p.A + (int64_t)(mb * 16 + ld_row) * p.K + kbeg + ld_grp * 16;
		const bool xvalid = mb * 16 + ld_row < p.M;
		sa[mb] = 0;
#pragma unroll
		for (int s = 0; s < SMAX; s++) {
			fx[mb][s] = zero_u8;  // what the sign flip turns into zeros: rows past M, k past the share
			if (xvalid && s * 64 + ld_grp * 16 < klen) fx[mb][s] = *reinterpret_cast<const v4i*>(xrow + s * 64);
		}
	}
	// the first row group's slab goes in flight behind the activations, so that the exchange below can wait for the
	// activations alone (loads complete in order) while the slab is still arriving
	issue_slab(blockIdx.x, 0);
	if (klen > 0) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
	else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
	if (exchange) {
		const int src = 4 * lrow + lgrp;  // the lane that fetched what this lane feeds to the MFMA
#pragma unroll
		for (int mb = 0; mb < MB; mb++)
#pragma unroll
			for (int s = 0; s < SMAX; s++) {
				fx[mb][s].x = __shfl(fx[mb][s].x, src, 64);
				fx[mb][s].y = __shfl(fx[mb][s].y, src, 64);
				fx[mb][s].z = __shfl(fx[mb][s].z, src, 64);
				fx[mb][s].w = __shfl(fx[mb][s].w, src, 64);
			}
	}
#pragma unroll
	for (int mb = 0; mb < MB; mb++) {
#pragma unroll
		for (int s = 0; s < SMAX; s++) {
			fx[mb][s] = flip_sign_bits(fx[mb][s]);
			if (SUM_A) {
				sa[mb] = __builtin_amdgcn_sdot4(fx[mb][s].x, 0x01010101, sa[mb], false);
				sa[mb] = __builtin_amdgcn_sdot4(fx[mb][s].y, 0x01010101, sa[mb], false);
				sa[mb] = __builtin_amdgcn_sdot4(fx[mb][s].z, 0x01010101, sa[mb], false);
				sa[mb] = __builtin_amdgcn_sdot4(fx[mb][s].w, 0x01010101, sa[mb], false);
			}
		}
		// a lane holds the sums of its 16-byte k-group only: fold the four k-groups (lanes l, l+16, l+32, l+48)
		if (SUM_A) {
			sa[mb] += __shfl_xor(sa[mb], 16, 64);
			sa[mb] += __shfl_xor(sa[mb], 32, 64);
			if (lane < 16) sums_a[wave][mb][lane] = sa[mb];  // the same for every row group: written once
		}
	}

	int parity = 0;
	for (int group = blockIdx.x; group < groups; group += gridDim.x, parity = (parity + 1) & (PAR - 1)) {
		v4i acc[MB];
#pragma unroll
		for (int mb = 0; mb < MB; mb++) acc[mb] = v4i{ 0, 0, 0, 0 };
		int sb = 0;
		// The bias of this row group is fetched here and taken into a register behind the wait for the slab: the compiler
		// waits for a load of its own before its first use, and behind the next slab's loads that wait would cover them too.
		int bias_n = 0;
		if (wave == 0 && bias && group * 16 + lrow < p.N) bias_n = bias[group * 16 + lrow];
#pragma unroll
		for (int pass = 0; pass < PASSES; pass++) {
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // own slab has landed (no other wave reads this slab)
			if (pass == 0) asm volatile("" : "+v"(bias_n));
#pragma unroll
			for (int s = 0; s < 16; s++) {
				const int gs = pass * 16 + s;
				if (gs < steps) {
					v4i fw = *reinterpret_cast<const v4i*>(wfrag + s * 64);
					fw = flip_bits(fw, p.b_flip);
					// the 16 bytes of a partial last step that lie past K were never loaded
					if (gs * 64 + lgrp * 16 >= klen) fw = v4i{ 0, 0, 0, 0 };
					if (SUM_B) {
						sb = __builtin_amdgcn_sdot4(fw.x, 0x01010101, sb, false);
						sb = __builtin_amdgcn_sdot4(fw.y, 0x01010101, sb, false);
						sb = __builtin_amdgcn_sdot4(fw.z, 0x01010101, sb, false);
						sb = __builtin_amdgcn_sdot4(fw.w, 0x01010101, sb, false);
					}
					// MFMA A operand = activations (rows m), B operand = weights (columns n):
					// lane (lrow, lgrp), register e holds out[m = mb*16 + 4*lgrp + e][n = lrow]
#pragma unroll
					for (int mb = 0; mb < MB; mb++) acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fx[mb][gs], fw, acc[mb], 0, 0, 0);
				}
			}
			// the slab is consumed (its values sit in registers): the next pass or the next row group's slab can start to arrive
			asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
			if (pass + 1 < PASSES) issue_slab(group, pass + 1);
			else if (group + (int)gridDim.x < groups) issue_slab(group + gridDim.x, 0);
		}
		if (SUM_B) {
			sb += __shfl_xor(sb, 16, 64); sb += __shfl_xor(sb, 32, 64);
			if (lane < 16) sums_b[parity][wave][lane] = sb;
		}
		// partial accumulators of the k-slices meet in LDS; the two parities keep wave 0's reads of one row
		// group apart from the other waves' writes of the next
#pragma unroll
		for (int mb = 0; mb < MB; mb++) *reinterpret_cast<v4i*>(&partial[parity][wave][mb][lane * 4]) = acc[mb];
		__syncthreads();
		if (wave != 0) {
			if (PAR == 1) __syncthreads();
			continue;
		}
		int tsb = 0;
		if (SUM_B) {
#pragma unroll
			for (int w = 0; w < WAVES; w++) tsb += sums_b[parity][w][lrow];
		}
		const int n = group * 16 + lrow;
		// sum a'b' -> l-ten's element: + coef_a * sum_k a' + coef_b * sum_k b' + K * coef_a * coef_b (+ bias)
		//   with a' = a - 128, coef_a = 128 - zpB, coef_b = 128 - zpA
		const int base = coef_b * tsb + (Kc - pad_here) * coef_a * coef_b + bias_n;
#pragma unroll
		for (int mb = 0; mb < MB; mb++) {
			v4i tot = { 0, 0, 0, 0 };
			int tsa[4] = { 0, 0, 0, 0 };
#pragma unroll
			for (int w = 0; w < WAVES; w++) {
				tot += *reinterpret_cast<const v4i*>(&partial[parity][w][mb][lane * 4]);
				if (SUM_A) {
#pragma unroll
					for (int e = 0; e < 4; e++) tsa[e] += sums_a[w][mb][lgrp * 4 + e];
				}
			}
#pragma unroll
			for (int e = 0; e < 4; e++) {
				const int m = mb * 16 + lgrp * 4 + e;
				if (m >= p.M || n >= p.N) continue;
				const int v = tot[e] + base + coef_a * tsa[e];
				if (OUT == Q_OUT_ACC) static_cast<int*>(p.C)[(int64_t)m * p.N + n] = v;
				else static_cast<uint8_t*>(p.C)[(int64_t)m * p.N + n] = (uint8_t)requant<OUT>(v, p.mult, p.zp_c);
			}
		}
		if (PAR == 1) __syncthreads();
	}
}

template <int WAVES, int SMAX, int MB>
static int launch_skinny(const QProblem& p, int out, const int32_t* bias, int coef_a, int coef_b, int kw, const char* name, int chunk_k = 0, int chunks = 1)
{
	// as many workgroups as fit the CUs' LDS at once (one per CU with eight wavefronts); each walks row groups blockIdx.x, blockIdx.x + grid, ...
	constexpr int PAR = MB == 1 ? 2 : 1;
	constexpr int LDS_BYTES = WAVES * 16 * (1024 + 16) + PAR * WAVES * MB * 1024 + (PAR + MB) * WAVES * 64;
	static_assert(LDS_BYTES <= 160 * 1024, "slabs and partial tiles must fit the CU's LDS");
	constexpr int PER_CU = (160 * 1024) / LDS_BYTES;
	const dim3 grid((unsigned)std::min<int64_t>((p.N + 15) / 16, std::max(1, 256 * PER_CU / chunks)), (unsigned)chunks), block(WAVES * 64);
	set_kernel_name(name);
	const bool sum_a = coef_a != 0, sum_b = coef_b != 0;
#define LTEN_SK(OUTV, SA, SB) qskinny_kernel<WAVES, SMAX, MB, OUTV, SA, SB><<<grid, block, 0, stream()>>>(p, bias, coef_a, coef_b, kw, chunk_k)
#define LTEN_SK_OUT(OUTV)                                     \
	if (sum_a && sum_b) LTEN_SK(OUTV, true, true);        \
	else if (sum_a) LTEN_SK(OUTV, true, false);           \
	else if (sum_b) LTEN_SK(OUTV, false, true);           \
	else LTEN_SK(OUTV, false, false);
#define LTEN_SK_CHUNKS(SA, SB) qskinny_kernel<WAVES, SMAX, MB, Q_OUT_ACC, SA, SB, true><<<grid, block, 0, stream()>>>(p, bias, coef_a, coef_b, kw, chunk_k)
	if (chunk_k != 0) {  // (only with int32 sums)
		if (out != Q_OUT_ACC) return -1;
		if (sum_a && sum_b) LTEN_SK_CHUNKS(true, true);
		else if (sum_a) LTEN_SK_CHUNKS(true, false);
		else if (sum_b) LTEN_SK_CHUNKS(false, true);
		else LTEN_SK_CHUNKS(false, false);
	}
	else if (out == Q_OUT_U8_FAST) { LTEN_SK_OUT(Q_OUT_U8_FAST) }
	else if (out == Q_OUT_U8_EXACT) { LTEN_SK_OUT(Q_OUT_U8_EXACT) }
	else { LTEN_SK_OUT(Q_OUT_ACC) }
#undef LTEN_SK_CHUNKS
#undef LTEN_SK_OUT
#undef LTEN_SK
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// out[i] = requantize(acc[0][i] + acc[1][i] + ...) (or the int32 sum itself): the K-chunks of a long reduction meet here
template <int OUT>
__global__ __launch_bounds__(256) void qskinny_sum_chunks_kernel(const int32_t* __restrict__ acc, int chunks, int64_t count, float mult, float zp_c, void* __restrict__ out)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= count) return;
	// (four loads in flight at a time)
	int v = 0, c = 0;
	for (; c + 4 <= chunks; c += 4) {
		int t[4];
#pragma unroll
		for (int j = 0; j < 4; j++) t[j] = acc[(int64_t)(c + j) * count + idx];
		v += (t[0] + t[1]) + (t[2] + t[3]);
	}
	for (; c < chunks; c++) v += acc[(int64_t)c * count + idx];
	if (OUT == Q_OUT_ACC) static_cast<int*>(out)[idx] = v;
	else static_cast<uint8_t*>(out)[idx] = (uint8_t)requant<OUT>(v, mult, zp_c);
}

// Returns -1 when the problem does not fit the streaming kernel (the caller then uses the other kernels): up to 32
// activation rows against weights with 16-byte aligned rows (K a multiple of 16), K up to 8192, or up to 16384 with at
// most 16 rows (the activations of a wavefront's share of K stay in registers).  N is arbitrary.
int qskinny_dispatch(const QProblem& p, int out, const int32_t* bias, int zp_a, int zp_b)
{
	if (!(p.a_ks == 1 && p.b_ks == 1 && p.vec_ok && p.M >= 1 && p.M <= 32 && p.N >= 1 && p.K >= 64)) return -1;
	const int coef_a = 128 - zp_b, coef_b = 128 - zp_a;
	const int k_whole = p.M > 16 ? 8192 : 16384;  // what one launch takes whole: the activations of a wavefront's share sit in registers
	// (also a K of 16384 against fewer than 128 groups of 16 weight rows, which would leave half of the CUs idle through two
	// slab passes: 1 x 1000 x 16384 12 us whole)
	if (p.K > k_whole || (p.K >= 16384 && p.N < 128 * 16)) {
		// A reduction longer than the registers of eight wavefronts hold the activations of (a 25088 -> 4096 layer at batch
		// 1; from 17 rows on, K above 8192): K in chunks, all in one launch (grid rows), each into int32 sums of its own in memory the library owns (the
		// identity's terms are sums over k, so the chunks' l-ten accumulators add up; the bias goes with the first), and a
		// second launch adds the chunks and requantizes.  As many chunks as give the chip about 512 workgroups with the
		// groups of 16 weight rows there are (a 1000-row layer has 63), of 2048 or more k each.
		const uint64_t groups = ceil_div((uint64_t)p.N, 16);
		int chunks = (int)std::max<uint64_t>(ceil_div((uint64_t)p.K, (uint64_t)k_whole), std::min<uint64_t>(16, ceil_div(512, groups)));
		while (chunks > 2 && p.K / chunks < 2048) chunks--;
		if ((uint64_t)p.K * 255 * 255 >= (1ull << 31)) return -1;
		const int ck = (int)ceil_div(ceil_div((uint64_t)p.K, (uint64_t)chunks), 64) * 64;
		chunks = (int)ceil_div((uint64_t)p.K, (uint64_t)ck);
		const int64_t count = (int64_t)p.M * p.N;
		int32_t* acc = static_cast<int32_t*>(library_scratch((uint64_t)chunks * count * sizeof(int32_t)));
		if (acc == nullptr) return -1;
		QProblem pc = p;
		pc.C = acc;
		const int wv = ck <= 2048 ? 2 : (ck <= 4096 ? 4 : 8);
		const int kwc = (int)ceil_div(ceil_div((uint64_t)ck, (uint64_t)wv), 64) * 64;
		int rc;
		if (p.M > 16) {  // two blocks of 16 activation rows, chunks of at most 8192
			if (wv == 8) rc = launch_skinny<8, 16, 2>(pc, Q_OUT_ACC, bias, coef_a, coef_b, kwc, "qskinny", ck, chunks);
			else if (wv == 4) rc = launch_skinny<4, 16, 2>(pc, Q_OUT_ACC, bias, coef_a, coef_b, kwc, "qskinny", ck, chunks);
			else rc = launch_skinny<2, 16, 2>(pc, Q_OUT_ACC, bias, coef_a, coef_b, kwc, "qskinny", ck, chunks);
		}
		else if (ck > 8192) rc = launch_skinny<8, 32, 1>(pc, Q_OUT_ACC, bias, coef_a, coef_b, kwc, "qskinny", ck, chunks);
		else if (wv == 8) rc = launch_skinny<8, 16, 1>(pc, Q_OUT_ACC, bias, coef_a, coef_b, kwc, "qskinny", ck, chunks);
		else if (wv == 4) rc = launch_skinny<4, 16, 1>(pc, Q_OUT_ACC, bias, coef_a, coef_b, kwc, "qskinny", ck, chunks);
		else rc = launch_skinny<2, 16, 1>(pc, Q_OUT_ACC, bias, coef_a, coef_b, kwc, "qskinny", ck, chunks);
		if (rc) return rc;
		const dim3 grid((unsigned)ceil_div((uint64_t)count, 256));
		if (out == Q_OUT_U8_FAST) qskinny_sum_chunks_kernel<Q_OUT_U8_FAST><<<grid, dim3(256), 0, stream()>>>(acc, chunks, count, p.mult, p.zp_c, p.C);
		else if (out == Q_OUT_U8_EXACT) qskinny_sum_chunks_kernel<Q_OUT_U8_EXACT><<<grid, dim3(256), 0, stream()>>>(acc, chunks, count, p.mult, p.zp_c, p.C);
		else qskinny_sum_chunks_kernel<Q_OUT_ACC><<<grid, dim3(256), 0, stream()>>>(acc, chunks, count, p.mult, p.zp_c, p.C);
		LTEN_HIP_LAUNCH_CHECK();
		set_kernel_name("qskinny_mfma_kchunks");
		return 0;
	}
	const int waves = p.K <= 2048 ? 2 : (p.K <= 4096 ? 4 : 8);
	const int kw = (int)ceil_div(ceil_div((uint64_t)p.K, (uint64_t)waves), 64) * 64;
	if (p.K > 8192) return launch_skinny<8, 32, 1>(p, out, bias, coef_a, coef_b, kw, "qskinny_mfma_w8_2pass");
	if (p.M <= 16) {
		if (waves == 8) return launch_skinny<8, 16, 1>(p, out, bias, coef_a, coef_b, kw, "qskinny_mfma_w8");
		if (waves == 4) return launch_skinny<4, 16, 1>(p, out, bias, coef_a, coef_b, kw, "qskinny_mfma_w4");
		return launch_skinny<2, 16, 1>(p, out, bias, coef_a, coef_b, kw, "qskinny_mfma_w2");
	}
	// two blocks of 16 activation rows against every weight fragment
	if (waves == 8) return launch_skinny<8, 16, 2>(p, out, bias, coef_a, coef_b, kw, "qskinny_mfma_w8_m32");
	if (waves == 4) return launch_skinny<4, 16, 2>(p, out, bias, coef_a, coef_b, kw, "qskinny_mfma_w4_m32");
	return launch_skinny<2, 16, 2>(p, out, bias, coef_a, coef_b, kw, "qskinny_mfma_w2_m32");
}

}  // namespace lten_hip
