// int8 GEMM for gfx950: the GPU counterpart of l-ten's quantized_matmul
// (l-ten/math_fns.cpp:1311-1478), which has no GPU implementation in l-ten
// (l-ten/fully_connected.cpp:399).
//
// Arithmetic.  l-ten multiplies two uint8 matrices with uint8 zero points.  The matrix
// cores multiply signed bytes, so every operand byte is mapped to a' = a XOR 0x80
// (= a - 128 as int8) on its way into LDS, and the exact integer identity
//
//   sum_k (A-zpA)(B-zpB) = sum_k a'b' + (128-zpB) * SA_m + (128-zpA) * SB_n + K (zpA zpB - 16384)
//
// (SA_m, SB_n = plain byte sums of row m of A / row n of B) restores l-ten's value
// `element` of :1469 in the epilogue, which then requantizes exactly as :1474 does.
// All integer arithmetic wraps modulo 2^32, which equals l-ten's int arithmetic wherever
// that does not overflow.
//
// Tiling.  One workgroup computes a BM x BN tile of C with WM x WN wavefronts; each
// wavefront owns a (BM/WM) x (BN/WN) sub-tile built from 32x32x32 int8 MFMA blocks.  The
// MFMA "A" operand is fed from the weight tile and the "B" operand from the activation
// tile, so that the four consecutive accumulator registers of a lane are four consecutive
// output columns n and are stored as one packed dword.  A and B tiles are staged through
// LDS in two buffers (global -> registers -> XOR -> LDS while the MFMAs of the current
// buffer run), rows of BK bytes with a 16-byte-chunk XOR swizzle that keeps the
// ds_read_b128 operand fetches bank-conflict free.
#include "common.h"
#include "qgemm_common.h"

#include <algorithm>

namespace lten_hip {

// One 16-byte chunk of an operand tile, raw bytes (before the XOR), as four dwords.
// Out-of-range bytes read as `pad` (0x80 for uint8 data), which becomes 0 after the XOR.
template <bool GUARD>
__device__ __forceinline__ v4i load_chunk(const uint8_t* base, int64_t rs, int64_t ks, int row, int rows, int k, int K, int vec_ok, unsigned pad)
{
	if (!GUARD) {
		return *reinterpret_cast<const v4i*>(base + (int64_t)row * rs + k);
	} else {
		if (ks == 1 && vec_ok && row < rows && k + 16 <= K)
			return *reinterpret_cast<const v4i*>(base + (int64_t)row * rs + k);
		v4i v;
		int* vp = reinterpret_cast<int*>(&v);
#pragma unroll
		for (int d = 0; d < 4; d++) {
			unsigned w = 0;
#pragma unroll
			for (int b = 0; b < 4; b++) {
				int kk = k + d * 4 + b;
				unsigned byte = pad;
				if (row < rows && kk < K) byte = base[(int64_t)row * rs + (int64_t)kk * ks];
				w |= byte << (8 * b);
			}
			vp[d] = (int)w;
		}
		return v;
	}
}

template <int BM, int BN, int BK, int WM, int WN, bool GUARD, int OUT>
__global__ __launch_bounds__(WM* WN * 64) void qgemm_kernel(QProblem p)
{
	constexpr int T = WM * WN * 64;
	constexpr int CPR = BK / 16;  // 16-byte chunks per tile row
	constexpr int TM = BM / WM, TN = BN / WN;
	constexpr int FM = TM / 32, FN = TN / 32;
	constexpr int A_CHUNKS = BM * CPR, B_CHUNKS = BN * CPR;
	constexpr int A_PER_T = (A_CHUNKS + T - 1) / T, B_PER_T = (B_CHUNKS + T - 1) / T;
	constexpr int STAGE = (BM + BN) * BK;
	static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA block");
	static_assert(BK % 32 == 0, "BK must hold whole MFMA k-slices");

	__shared__ __attribute__((aligned(16))) uint8_t smem[2 * STAGE];

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int wm = wave / WN, wn = wave % WN;

	// Workgroup -> tile.  Consecutive workgroup ids go round-robin to the 8 XCDs, each
	// with its own L2; give every XCD one compact block of tiles so that the A rows and
	// B rows it streams are shared by its CUs.
	const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
	int bid = blockIdx.x;
	int tm, tn;
	{
		const int nb = tiles_m * tiles_n;
		int lid = bid;
		if ((nb & 7) == 0) lid = (bid & 7) * (nb >> 3) + (bid >> 3);
		constexpr int GM = 4, GN = 8;
		if (tiles_m % GM == 0 && tiles_n % GN == 0) {
			int group = lid / (GM * GN), within = lid % (GM * GN);
			int groups_n = tiles_n / GN;
			tm = (group / groups_n) * GM + within / GN;
			tn = (group % groups_n) * GN + within % GN;
		} else {
			tm = lid / tiles_n;
			tn = lid % tiles_n;
		}
	}
	const int m0 = tm * BM, n0 = tn * BN;

	const bool a_kmajor = (p.a_ks == 1), b_kmajor = (p.b_ks == 1);

	v4i stage_a[A_PER_T], stage_b[B_PER_T];

	auto load_global = [&](int k0) {
#pragma unroll
		for (int i = 0; i < A_PER_T; i++) {
			int c = tid + i * T;
			if (A_CHUNKS % T != 0 && c >= A_CHUNKS) break;
			// K-contiguous operands: neighbouring threads take neighbouring chunks of a row.
			// K-strided operands: neighbouring threads take neighbouring rows.
			int row = (!GUARD || a_kmajor) ? c / CPR : c % BM;
			int kc = (!GUARD || a_kmajor) ? c % CPR : c / BM;
			stage_a[i] = load_chunk<GUARD>(p.A, p.a_rs, p.a_ks, m0 + row, p.M, k0 + kc * 16, p.K, p.vec_ok, 0x80u);
		}
#pragma unroll
		for (int i = 0; i < B_PER_T; i++) {
			int c = tid + i * T;
			if (B_CHUNKS % T != 0 && c >= B_CHUNKS) break;
			int row = (!GUARD || b_kmajor) ? c / CPR : c % BN;
			int kc = (!GUARD || b_kmajor) ? c % CPR : c / BN;
			stage_b[i] = load_chunk<GUARD>(p.B, p.b_rs, p.b_ks, n0 + row, p.N, k0 + kc * 16, p.K, p.vec_ok, p.b_flip & 0xffu);
		}
	};

	auto store_lds = [&](int buf) {
		uint8_t* sa = smem + buf * STAGE;
		uint8_t* sb = sa + BM * BK;
#pragma unroll
		for (int i = 0; i < A_PER_T; i++) {
			int c = tid + i * T;
			if (A_CHUNKS % T != 0 && c >= A_CHUNKS) break;
			int row = (!GUARD || a_kmajor) ? c / CPR : c % BM;
			int kc = (!GUARD || a_kmajor) ? c % CPR : c / BM;
			*reinterpret_cast<v4i*>(sa + row * BK + ((kc ^ swz<CPR>(row)) << 4)) = flip_sign_bits(stage_a[i]);
		}
#pragma unroll
		for (int i = 0; i < B_PER_T; i++) {
			int c = tid + i * T;
			if (B_CHUNKS % T != 0 && c >= B_CHUNKS) break;
			int row = (!GUARD || b_kmajor) ? c / CPR : c % BN;
			int kc = (!GUARD || b_kmajor) ? c % CPR : c / BN;
			*reinterpret_cast<v4i*>(sb + row * BK + ((kc ^ swz<CPR>(row)) << 4)) = flip_bits(stage_b[i], p.b_flip);
		}
	};

	v16i acc[FN][FM];
#pragma unroll
	for (int i = 0; i < FN; i++)
#pragma unroll
		for (int j = 0; j < FM; j++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

	const int KT = (p.K + BK - 1) / BK;
	const int lrow = lane & 31;  // row of the 32-row MFMA operand block this lane feeds
	const int lgrp = lane >> 5;  // which 16-byte half of the 32-byte k-slice

	load_global(0);
	store_lds(0);
	__syncthreads();

	for (int kt = 0; kt < KT; kt++) {
		const int cur = kt & 1;
		if (kt + 1 < KT) load_global((kt + 1) * BK);

		const uint8_t* sa = smem + cur * STAGE;
		const uint8_t* sb = sa + BM * BK;
#pragma unroll
		for (int s = 0; s < BK / 32; s++) {
			v4i fw[FN], fx[FM];
			const int kc = s * 2 + lgrp;
#pragma unroll
			for (int i = 0; i < FN; i++) {
				int row = wn * TN + i * 32 + lrow;
				fw[i] = *reinterpret_cast<const v4i*>(sb + row * BK + ((kc ^ swz<CPR>(row)) << 4));
			}
#pragma unroll
			for (int j = 0; j < FM; j++) {
				int row = wm * TM + j * 32 + lrow;
				fx[j] = *reinterpret_cast<const v4i*>(sa + row * BK + ((kc ^ swz<CPR>(row)) << 4));
			}
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int j = 0; j < FM; j++)
					acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[i], fx[j], acc[i][j], 0, 0, 0);
		}

		if (kt + 1 < KT) store_lds(cur ^ 1);
		__syncthreads();
	}

	// Epilogue.  Lane (lrow, lgrp) of block (i, j) holds, in register 4q + e, the output
	// at m = m0 + wm*TM + j*32 + lrow, n = n0 + wn*TN + i*32 + 8q + 4*lgrp + e.
#pragma unroll
	for (int j = 0; j < FM; j++) {
		const int m = m0 + wm * TM + j * 32 + lrow;
		if (GUARD && m >= p.M) continue;
		const int rt = (p.rterm ? p.rterm[m] : 0) + p.konst;
#pragma unroll
		for (int i = 0; i < FN; i++) {
#pragma unroll
			for (int q = 0; q < 4; q++) {
				const int n = n0 + wn * TN + i * 32 + q * 8 + lgrp * 4;
				int v[4];
#pragma unroll
				for (int e = 0; e < 4; e++) {
					v[e] = acc[i][j][q * 4 + e] + rt;
					if (p.cterm && (!GUARD || n + e < p.N)) v[e] += p.cterm[n + e];
				}
				if (OUT == Q_OUT_ACC) {
					int* out = static_cast<int*>(p.C) + (int64_t)m * p.N + n;
					if (!GUARD) {
						*reinterpret_cast<v4i*>(out) = v4i{ v[0], v[1], v[2], v[3] };
					} else {
#pragma unroll
						for (int e = 0; e < 4; e++)
							if (n + e < p.N) out[e] = v[e];
					}
				} else {
					unsigned b0 = requant<OUT>(v[0], p.mult, p.zp_c);
					unsigned b1 = requant<OUT>(v[1], p.mult, p.zp_c);
					unsigned b2 = requant<OUT>(v[2], p.mult, p.zp_c);
					unsigned b3 = requant<OUT>(v[3], p.mult, p.zp_c);
					uint8_t* out = static_cast<uint8_t*>(p.C) + (int64_t)m * p.N + n;
					if (!GUARD) {
						*reinterpret_cast<unsigned*>(out) = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
					} else {
						if (n + 0 < p.N) out[0] = (uint8_t)b0;
						if (n + 1 < p.N) out[1] = (uint8_t)b1;
						if (n + 2 < p.N) out[2] = (uint8_t)b2;
						if (n + 3 < p.N) out[3] = (uint8_t)b3;
					}
				}
			}
		}
	}
}

// Byte sums of the rows of A and of B, turned into the epilogue's correction vectors:
//   rterm[m] = (128 - zpB) * sum_k A[m,k]
//   cterm[n] = (128 - zpA) * sum_k B[n,k] + bias[n]
// One wavefront per row; a zero coefficient skips the read of that matrix.
__global__ __launch_bounds__(256) void qgemm_terms_kernel(QProblem p, int coef_a, int coef_b, const int32_t* bias,
                                                          int32_t* rterm, int32_t* cterm)
{
	const int lane = threadIdx.x & 63;
	const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	const bool is_a = wave < p.M;
	const int64_t row = is_a ? wave : wave - p.M;
	if (!is_a && row >= p.N) return;
	const uint8_t* base = is_a ? p.A : p.B;
	const int64_t rs = is_a ? p.a_rs : p.b_rs, ks = is_a ? p.a_ks : p.b_ks;
	const int coef = is_a ? coef_a : coef_b;
	const unsigned unflip = is_a ? 0u : (0x80808080u ^ p.b_flip);  // prepared weights hold b ^ 0x80
	unsigned sum = 0;
	if (coef != 0) {
		const uint8_t* r = base + row * rs;
		if (ks == 1 && p.vec_ok) {
			int k = lane * 16;
			for (; k + 16 <= p.K; k += 64 * 16) {
				v4i v = *reinterpret_cast<const v4i*>(r + k);
				const unsigned one = 0x01010101u;
				sum = __builtin_amdgcn_udot4((unsigned)v.x ^ unflip, one, sum, false);
				sum = __builtin_amdgcn_udot4((unsigned)v.y ^ unflip, one, sum, false);
				sum = __builtin_amdgcn_udot4((unsigned)v.z ^ unflip, one, sum, false);
				sum = __builtin_amdgcn_udot4((unsigned)v.w ^ unflip, one, sum, false);
			}
			// tail shorter than 16 bytes: the lane whose chunk straddles K finishes it
			if (k < p.K)
				for (int kk = k; kk < p.K && kk < k + 16; kk++) sum += r[kk] ^ (unflip & 0xffu);
		} else {
			for (int k = lane; k < p.K; k += 64) sum += r[(int64_t)k * ks] ^ (unflip & 0xffu);
		}
#pragma unroll
		for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off, 64);
	}
	if (lane == 0) {
		if (is_a)
			rterm[row] = (int)(sum * (unsigned)coef);
		else
			cterm[row] = (int)(sum * (unsigned)coef) + (bias ? bias[row] : 0);
	}
}

// -------------------------------------------------------------------------- dispatch

template <int BM, int BN, int BK, int WM, int WN, bool GUARD>
static int launch_tile(const QProblem& p, int out, const char* name)
{
	const unsigned grid = (unsigned)(ceil_div(p.M, BM) * ceil_div(p.N, BN));
	const dim3 block(WM * WN * 64);
	set_kernel_name(name);
	switch (out) {
	case Q_OUT_U8_FAST:
		qgemm_kernel<BM, BN, BK, WM, WN, GUARD, Q_OUT_U8_FAST><<<dim3(grid), block, 0, stream()>>>(p);
		break;
	case Q_OUT_U8_EXACT:
		qgemm_kernel<BM, BN, BK, WM, WN, GUARD, Q_OUT_U8_EXACT><<<dim3(grid), block, 0, stream()>>>(p);
		break;
	default:
		qgemm_kernel<BM, BN, BK, WM, WN, GUARD, Q_OUT_ACC><<<dim3(grid), block, 0, stream()>>>(p);
		break;
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// fast_only: try the direct-to-LDS tiles alone and return -1 when none of them takes the problem (the caller then
// prepares the zero-point vectors the general kernels need and calls again).
static int qgemm_dispatch(const QProblem& p, int out, const SplitScratch* scratch, bool fast_only = false)
{
	const bool kmajor = p.a_ks == 1 && p.b_ks == 1;
	const bool c_ok = (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
	auto fits = [&](int bm, int bn, int bk) {
		return kmajor && p.vec_ok && c_ok && p.M % bm == 0 && p.N % bn == 0 && p.K % bk == 0;
	};
	const uint64_t out_elems = (uint64_t)p.M * p.N;
	int choice = get_option(OPT_QGEMM_TILE);  // 0 = heuristic
	if (choice == 0) {
		// Problems that tile exactly go to the direct-to-LDS kernels when K is long enough to amortise their prologue
		// and epilogue: 256x256 tiles once those occupy most of the 256 CUs, 128x128 tiles (up to four times as many
		// workgroups, two per CU) below that.
		// (a shorter K only with many tiles: the positions x channels products of a quantized convolution, 16384 x 64 x
		// 288: 5.6 against 7.8 us on the guarded kernel)
		// (down to K = 32, one partial k-step: 2048 x 8192 x 64 took 42 us on the register-staged 256 x 256 tiles, 10 us here;
		// 4096 x 4096 x 96 53 -> 9.5 us)
		if (p.K >= 512 || (p.K >= 32 && ceil_div(p.M, 128) * ceil_div(p.N, 128) >= 64)) {
			// 256 x 256 tiles only where both dimensions fill most of one (100352 x 64 x 576: 20.7 us on 128 x 128 tiles, 26.5 on these)
			if (p.M >= 192 && p.N >= 192 && ceil_div(p.M, 256) * ceil_div(p.N, 256) > 160 && qgemm_fast_dispatch(p, out, 33) == 0) return 0;
			// about one 256 x 128 tile per CU: less operand traffic per MFMA than two 128 x 128 tiles per CU
			const uint64_t tiles_256x128 = ceil_div(p.M, 256) * ceil_div(p.N, 128);
			if (tiles_256x128 > 160 && tiles_256x128 <= 256 && p.K >= 2048 && qgemm_fast_dispatch(p, out, 51) == 0) return 0;
			// Outputs that give 128 x 128 tiles to at most a quarter of the CUs, with a long K: several workgroups share a
			// tile, each with a slice of K (option "qgemm_split": 0 automatic, 1 off, 2 / 4 / 8 forced).  The exchange of
			// partial sums between workgroups is dear on this part, so the split pays only there: 1024 x 4096 weights
			// at M = 256 16.5 -> 14.0 us, 8192 x 8192 at M = 128 30.4 -> 25.6 us, but 4096 x 4096 at M = 256 17.3 -> 19.0
			// us and at M = 512 17.5 -> 26.5 us.
			const int want = get_option(OPT_QGEMM_SPLIT);
			const uint64_t tiles = ceil_div(p.M, 128) * ceil_div(p.N, 128);
			int splits = 1;
			if (want >= 2) splits = want;
			else if (want == 0 && tiles <= 64 && p.K >= 8192) splits = tiles <= 32 ? 4 : 2;
			else if (want == 0 && tiles <= 32 && p.K >= 4096) splits = 2;
			// (slices are whole k-steps of 128, the first ones a step longer when the slices do not divide them: 128 x 4096 x
			// 11008, 86 k-steps, 38 us unsplit, 27 in four slices)
			if (splits >= 2 && qgemm_fast_split_dispatch(p, out, splits, scratch) == 0) return 0;
			if (qgemm_fast_dispatch(p, out, 41) == 0) return 0;
		}
		if (fast_only) return -1;
		if (fits(256, 256, 64) && out_elems >= 256ull * 256 * 192)
			choice = 1;
		else if (fits(128, 128, 64) && out_elems >= 128ull * 128 * 128)
			choice = 2;
		else if (out_elems >= 64ull * 64 * 256)
			choice = 3;
		else
			choice = 4;
	}
	if (choice >= 20) {
		const int rc = qgemm_fast_dispatch(p, out, choice);
		if (fast_only) return rc;
		LTEN_HIP_REQUIRE(rc >= 0, "qgemm: forced fast variant %d does not fit this problem", choice);
		return rc;
	}
	if (fast_only) return -1;
	switch (choice) {
	case 1:
		LTEN_HIP_REQUIRE(fits(256, 256, 64), "qgemm: forced 256x256x64 tile does not fit this problem");
		return launch_tile<256, 256, 64, 2, 2, false>(p, out, "qgemm_nt_256x256x64");
	case 2:
		LTEN_HIP_REQUIRE(fits(128, 128, 64), "qgemm: forced 128x128x64 tile does not fit this problem");
		return launch_tile<128, 128, 64, 2, 2, false>(p, out, "qgemm_nt_128x128x64");
	case 3:
		return launch_tile<64, 64, 64, 2, 2, true>(p, out, "qgemm_guard_64x64x64");
	default:
		return launch_tile<32, 32, 64, 1, 1, true>(p, out, "qgemm_guard_32x32x64");
	}
}

// Scratch for an entry point that must not allocate: the zero-point terms (instead of the caller's workspace) and the
// split-K buffers (instead of the library's own, which are allocated on first use).
struct RunScratch {
	int32_t* terms;      // terms_ints ints
	uint64_t terms_ints;
	SplitScratch split;
};

// Rows of any length and alignment to rows of Kp bytes (a multiple of 16, so 16-byte aligned where dst is): one thread
// per 16 bytes of dst; bytes K .. Kp - 1 of a row become 128, the byte that reads as zero once the operands are
// taken as a - 128.  Rows 0 .. rows_a - 1 come from src_a, the others from src_b (the two operands of one product in
// one launch).  A dword of a row is put together from the two aligned dwords that hold it, whatever the row's
// alignment; only the dword that straddles the row's end is read byte by byte.
__global__ __launch_bounds__(256) void qgemm_pad_rows_kernel(const uint8_t* __restrict__ src_a, uint8_t* __restrict__ dst_a, uint64_t rows_a,
                                                             const uint8_t* __restrict__ src_b, uint8_t* __restrict__ dst_b, uint64_t rows_b, int K, int Kp)
{
	const uint64_t cpr = (uint64_t)Kp / 16, total = (rows_a + rows_b) * cpr;
	for (uint64_t c = (uint64_t)blockIdx.x * 256 + threadIdx.x; c < total; c += (uint64_t)gridDim.x * 256) {
		uint64_t row = c / cpr;
		const int k0 = (int)(c - row * cpr) * 16;
		const uint8_t* src = src_a;
		uint8_t* dst = dst_a;
		if (row >= rows_a) {
			row -= rows_a;
			src = src_b;
			dst = dst_b;
		}
		const uint8_t* r = src + row * (uint64_t)K;
		uint32_t v[4];
#pragma unroll
		for (int j = 0; j < 4; j++) {
			const int k = k0 + 4 * j;
			v[j] = 0x80808080u;
			if (k + 4 <= K) {
				const uintptr_t a = reinterpret_cast<uintptr_t>(r + k);
				const uint32_t* al = reinterpret_cast<const uint32_t*>(a & ~(uintptr_t)3);
				const unsigned sh = (unsigned)(a & 3);
				const uint32_t lo = al[0], hi = al[sh ? 1 : 0];  // all four bytes lie inside the row, so both dwords hold some of them
				v[j] = __builtin_amdgcn_alignbyte(hi, lo, sh);
			} else if (k < K) {
#pragma unroll
				for (int b = 0; b < 3; b++)
					if (k + b < K) v[j] = (v[j] & ~(0xFFu << (8 * b))) | ((uint32_t)r[k + b] << (8 * b));
			}
		}
		*reinterpret_cast<v4i*>(dst + row * (uint64_t)Kp + k0) = v4i{ (int)v[0], (int)v[1], (int)v[2], (int)v[3] };
	}
}

// An operand that lies with K as its outer index (src[k * R + r]: a transposed A, or B as quantized_matmul(.., false, ..)
// takes it) to rows of Kp bytes contiguous in K, padded with 128 as above: tiles of 64 x 64 bytes through LDS, read
// along r, written along k.
__global__ __launch_bounds__(256) void qgemm_transpose_rows_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int R, int K, int Kp)
{
	__shared__ __attribute__((aligned(16))) uint8_t tile[64][68];  // [r][k]
	const int tid = threadIdx.x, r0 = (int)blockIdx.x * 64, k0 = (int)blockIdx.y * 64;
	const bool dwords = (R & 3) == 0 && (reinterpret_cast<uintptr_t>(src) & 3) == 0;  // four r of a k in one aligned load
#pragma unroll
	for (int i = 0; i < 4; i++) {
		const int k = tid / 16 + 16 * i, r = 4 * (tid % 16);
		uint32_t v = 0x80808080u;
		if (k0 + k < K) {
			const uint8_t* p = src + (int64_t)(k0 + k) * R + r0 + r;
			if (dwords && r0 + r + 4 <= R) v = *reinterpret_cast<const uint32_t*>(p);
			else {
#pragma unroll
				for (int e = 0; e < 4; e++)
					if (r0 + r + e < R) v = (v & ~(0xFFu << (8 * e))) | ((uint32_t)p[e] << (8 * e));
			}
		}
#pragma unroll
		for (int e = 0; e < 4; e++) tile[r + e][k] = (uint8_t)(v >> (8 * e));
	}
	__syncthreads();
#pragma unroll
	for (int i = 0; i < 4; i++) {
		const int r = tid / 16 + 16 * i, k = 4 * (tid % 16);
		if (r0 + r < R && k0 + k < Kp) *reinterpret_cast<uint32_t*>(dst + (int64_t)(r0 + r) * Kp + k0 + k) = *reinterpret_cast<const uint32_t*>(&tile[r][k]);
	}
}

// k_pad: the last k_pad bytes of every row of A and B are padding (QProblem::k_pad); the call that pads passes it
static int qgemm_run(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, const uint8_t* A, const uint8_t* B, void* C,
                     int out_acc, const lten_hip_qparams* qp, const int32_t* bias, int32_t* workspace,
                     bool weights_prepared = false, const RunScratch* scratch = nullptr, const int32_t* weight_sums = nullptr, int k_pad = 0)
{
	LTEN_HIP_REQUIRE(qp != nullptr, "quantized_matmul: qparams is null");
	if (M == 0 || N == 0) return 0;
	LTEN_HIP_REQUIRE(A && B && C, "quantized_matmul: null matrix pointer");
	LTEN_HIP_REQUIRE(M < (1ull << 31) && N < (1ull << 31) && K < (1ull << 31), "quantized_matmul: dimension too large");
	// The reference accumulates u8*u8 products in int (l-ten/math_fns.cpp:1442-1467): beyond this K
	// it overflows and there is nothing defined to match.
	LTEN_HIP_REQUIRE(K * 65025ull < (1ull << 31), "quantized_matmul: K=%llu overflows the reference's int accumulator",
	                 (unsigned long long)K);

	// Rows that are no multiple of 16 bytes long (a layer of 1000 or 50 inputs) fit none of the kernels that load 16
	// bytes at a time, which is all but the guarded one: 4096 x 4096 x 4100 took 2.4 ms there where K = 4096 takes 56 us,
	// one row against 4096 x 4100 weights 197 us against 5.  The same holds for operands that lie with K as the outer
	// index (a transposed A; B as quantized_matmul(.., false, ..) takes it, which is how l-ten's Conv2d_q calls it).
	// Such products run on copies in the layout the layers use (both operands contiguous in K, rows padded to a
	// multiple of 16 bytes): one more launch per operand that needs it, then the kernels of the padded shape.  Prepared
	// weights are padded already (lten_hip_fcq_prepare_weights), so only the activations are copied.  The entry point
	// that may not allocate keeps the guarded kernel, and so do products too small to care (20 x 64 x 250, one image of
	// l-ten's quantized MNIST conv2 as l-ten multiplies it: 24 us on the guarded kernel, 8 us this way).
	const bool layer_layout = !tA && tB;
	if (k_pad == 0 && (!layer_layout || (K & 15) != 0) && scratch == nullptr && (weights_prepared || M * N * K >= (1ull << 16))) {
		const uint64_t Kp = (K + 15) & ~15ull;
		const bool copy_a = tA || Kp != K, copy_b = !weights_prepared && (!tB || Kp != K);
		const uint64_t bytes_a = copy_a ? M * Kp : 0, bytes_b = copy_b ? N * Kp : 0;
		uint8_t* buf = static_cast<uint8_t*>(library_scratch(bytes_a + bytes_b));
		LTEN_HIP_REQUIRE(buf != nullptr || !weights_prepared,
		                 "quantized_matmul: no memory for the padded copy of the activations (in_features = %llu is no multiple of 16; while a "
		                 "launch graph is being recorded the copy's memory cannot be allocated: run the call once before recording)",
		                 (unsigned long long)K);
		if (buf != nullptr) {
			uint8_t* const a2 = buf;
			uint8_t* const b2 = buf + bytes_a;
			// operands contiguous in K: both in one launch
			const uint64_t rows_a = copy_a && !tA ? M : 0, rows_b = copy_b && tB ? N : 0;
			if (rows_a + rows_b > 0) {
				const uint64_t chunks = (rows_a + rows_b) * (Kp / 16);
				const unsigned blocks = (unsigned)std::min<uint64_t>(ceil_div(chunks, 256), 16384);
				qgemm_pad_rows_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(A, a2, rows_a, B, b2, rows_b, (int)K, (int)Kp);
				LTEN_HIP_LAUNCH_CHECK();
			}
			if (tA) {
				qgemm_transpose_rows_kernel<<<dim3((unsigned)ceil_div(M, 64), (unsigned)(Kp / 64 + (Kp % 64 != 0))), dim3(256), 0, stream()>>>(A, a2, (int)M, (int)K, (int)Kp);
				LTEN_HIP_LAUNCH_CHECK();
			}
			if (copy_b && !tB) {
				qgemm_transpose_rows_kernel<<<dim3((unsigned)ceil_div(N, 64), (unsigned)(Kp / 64 + (Kp % 64 != 0))), dim3(256), 0, stream()>>>(B, b2, (int)N, (int)K, (int)Kp);
				LTEN_HIP_LAUNCH_CHECK();
			}
			// (a kernel choice that takes library memory of its own, the K-chunks of the streaming kernel, gets it behind the copies)
			LibraryScratchHold copies(bytes_a + bytes_b);
			return qgemm_run(0, 1, M, N, Kp, copy_a ? a2 : A, copy_b ? b2 : B, C, out_acc, qp, bias, workspace, weights_prepared, nullptr, weight_sums,
			                 (int)(Kp - K));
		}
	}

	const int zpA = qp[0].zero_point, zpB = qp[1].zero_point;
	QProblem p;
	p.A = A;
	p.B = B;
	p.C = C;
	// l-ten/math_fns.cpp:1445-1465: A is [M x K] or, transposed, [K x M]; B is [K x N] or, transposed, [N x K].
	p.a_rs = tA ? 1 : (int64_t)K;
	p.a_ks = tA ? (int64_t)M : 1;
	p.b_rs = tB ? (int64_t)K : 1;
	p.b_ks = tB ? 1 : (int64_t)N;
	p.M = (int)M;
	p.N = (int)N;
	p.K = (int)K;
	// With k_pad padding bytes of 128 in every row, byte sums over whole rows hold 128 k_pad too much each: taken off
	// here once for both sum terms (wrapping arithmetic, as the accumulators)
	p.k_pad = k_pad;
	p.konst = (int32_t)((uint32_t)(K - k_pad) * (uint32_t)(zpA * zpB - 16384) - (uint32_t)(128 * k_pad) * (uint32_t)((128 - zpB) + (128 - zpA)));
	// l-ten/math_fns.cpp:1436, left to right in fp32
	volatile float ab = qp[0].scale * qp[1].scale;
	p.mult = ab / qp[2].scale;
	p.zp_c = (float)qp[2].zero_point;
	p.b_flip = weights_prepared ? 0u : 0x80808080u;
	p.split_partial = nullptr;
	p.split_counters = nullptr;
	p.splits = 1;
	p.vec_ok = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 && (K & 15) == 0 &&
	           p.a_ks == 1 && p.b_ks == 1;

	int out = Q_OUT_ACC;
	if (!out_acc) {
		// |mult * acc + zp| < 2^31 for every int32 acc  <=>  the saturating GPU convert and the
		// x86 convert agree; otherwise take the epilogue that spells out the x86 behaviour.
		const float m = p.mult;
		out = (m == m && (m < 0 ? -m : m) <= 0.99f) ? Q_OUT_U8_FAST : Q_OUT_U8_EXACT;
	}

	// skinny activations: one streaming pass over the weights (option "qskinny": 0 = auto, 2 = off)
	p.cterm = nullptr;
	p.rterm = nullptr;
	const bool may_stream = get_option(OPT_QSKINNY) != 2 && get_option(OPT_QGEMM_TILE) == 0 && get_option(OPT_QGEMM_SPLIT) < 2;  // (a forced tile or split goes to the tiles)
	// below a megabyte of weights the one-launch kernel's many small workgroups win (option "qskinny" 1: stream anyway)
	const bool large_weights = N * K >= (1ull << 20) || get_option(OPT_QSKINNY) == 1;
	if (M <= 32 && large_weights && may_stream) {
		const int rc = qskinny_dispatch(p, out, bias, zpA, zpB);
		if (rc >= 0) return rc;
	}
	// (33 to 64 rows used to take two streaming passes, 32 rows and the rest; the 128 x 128 tiles with their split K have
	// since overtaken that: 64 x 4096 x 4096 15.3 against 18.0 us, 64 x 8192 x 8192 25.4 against 32.3 us, 40 x 11008 x
	// 4096 17.5 against 24.2 us)
	// small outputs: one launch that also takes the zero-point sums (same option switches it off)
	if (may_stream) {
		int rc = qdirect_dispatch(p, out, bias, zpA, zpB);
		if (rc >= 0) return rc;
		// few rows against weights that kernel does not take: still one streaming launch rather than the tiled kernels
		if (M <= 32) {
			rc = qskinny_dispatch(p, out, bias, zpA, zpB);
			if (rc >= 0) return rc;
		}
	}

	const int coef_a = 128 - zpB, coef_b = 128 - zpA;
	// Prepared weights come with their byte sums: the tiled kernels then work out every zero-point term themselves
	// and this call is one launch.
	if (weights_prepared && weight_sums != nullptr && (coef_a != 0 || coef_b != 0 || bias != nullptr)) {
		QProblem f = p;
		f.wsum = weight_sums;
		f.bias = bias;
		f.coef_a = coef_a;
		f.coef_b = coef_b;
		f.konst = (int32_t)((uint32_t)p.konst + (uint32_t)(128 * k_pad) * (uint32_t)coef_b);  // the kept weight sums count no padding
		if (qgemm_dispatch(f, out, scratch ? &scratch->split : nullptr, true) == 0) return 0;
	}
	if (coef_a != 0 || coef_b != 0 || bias != nullptr) {
		if (scratch != nullptr) {
			LTEN_HIP_REQUIRE(M + N <= scratch->terms_ints, "quantized_matmul: M + N = %llu exceeds the %llu rows and columns the static scratch holds",
			                 (unsigned long long)(M + N), (unsigned long long)scratch->terms_ints);
			workspace = scratch->terms;
		}
		LTEN_HIP_REQUIRE(workspace != nullptr, "quantized_matmul: workspace is null");
		p.cterm = workspace;      // N ints, where l-ten keeps row_vector (:1325)
		p.rterm = workspace + N;  // M ints, where l-ten keeps col_vector (:1326)
		const unsigned blocks = (unsigned)ceil_div(M + N, 4);
		qgemm_terms_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(p, coef_a, coef_b, bias, workspace + N, workspace);
		LTEN_HIP_LAUNCH_CHECK();
	}
	return qgemm_dispatch(p, out, scratch ? &scratch->split : nullptr);
}

__global__ __launch_bounds__(256) void fcq_prepare_weights_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, uint64_t n16,
                                                                  const uint8_t* __restrict__ src_tail, uint8_t* __restrict__ dst_tail, int tail)
{
	for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256) dst[i] = flip_sign_bits(src[i]);
	if (blockIdx.x == 0 && (int)threadIdx.x < tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x] ^ 0x80;
}

// The same conversion row by row, with each weight row's byte sum (of the uint8 values, as l-ten/math_fns.cpp:1364-1369
// adds them up on every call) kept in sums[row] (when not null): one wavefront per row.  Rows of dst are dst_cols
// bytes apart (cols rounded up to a multiple of 16); the bytes past cols become 0, the int8 form of the byte 128.
__global__ __launch_bounds__(256) void fcq_prepare_weights_sums_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int32_t* __restrict__ sums,
                                                                       uint64_t rows, uint64_t cols, uint64_t dst_cols, int vec_ok)
{
	const int lane = threadIdx.x & 63;
	const uint64_t row = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= rows) return;
	const uint8_t* r = src + row * cols;
	uint8_t* w = dst + row * dst_cols;
	unsigned sum = 0;
	uint64_t k = 0;
	if (vec_ok) {
		for (k = (uint64_t)lane * 16; k + 16 <= cols; k += 64 * 16) {
			const v4i v = *reinterpret_cast<const v4i*>(r + k);
			const unsigned one = 0x01010101u;
			sum = __builtin_amdgcn_udot4((unsigned)v.x, one, sum, false);
			sum = __builtin_amdgcn_udot4((unsigned)v.y, one, sum, false);
			sum = __builtin_amdgcn_udot4((unsigned)v.z, one, sum, false);
			sum = __builtin_amdgcn_udot4((unsigned)v.w, one, sum, false);
			*reinterpret_cast<v4i*>(w + k) = flip_sign_bits(v);
		}
		k = cols / 16 * 16;  // what is left of the row: fewer than 16 bytes
	}
	for (uint64_t kk = k + lane; kk < cols; kk += 64) {
		const uint8_t b = r[kk];
		sum += b;
		w[kk] = b ^ 0x80;
	}
	if (cols + lane < dst_cols) w[cols + lane] = 0;  // fewer than 16 bytes of padding
#pragma unroll
	for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off, 64);
	if (lane == 0 && sums != nullptr) sums[row] = (int32_t)sum;
}

// Scratch of lten_hip_fcq_forward_static: device memory that exists from the moment the library is loaded, so the
// entry point never allocates.  One copy per GPU (every device the code object is loaded on holds its own); the
// array's name is only a host-side handle, its device address comes from hipGetSymbolAddress.
constexpr uint64_t STATIC_TERMS_INTS = 64 * 1024;             // M + N of one call
constexpr uint64_t STATIC_SPLIT_BYTES = 8u << 20;             // partial sums of a split-K launch
constexpr int STATIC_SPLIT_TILES = 1024;
constexpr uint64_t STATIC_SCRATCH_BYTES = STATIC_SPLIT_BYTES + STATIC_TERMS_INTS * 4 + STATIC_SPLIT_TILES * 4;
static __device__ __align__(256) unsigned char fcq_static_scratch[STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 8;  // l-ten/globals.h:15
static unsigned char* g_static_scratch[MAX_DEVICES] = { nullptr };

// Device address of the current device's copy of the array, looked up once per device.
static int static_scratch(RunScratch* rs)
{
	int dev = -1;
	LTEN_HIP_CHECK(hipGetDevice(&dev));
	LTEN_HIP_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "lten_hip_fcq_forward_static: device %d out of range", dev);
	if (g_static_scratch[dev] == nullptr) {
		void* ptr = nullptr;
		LTEN_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(fcq_static_scratch)));
		LTEN_HIP_REQUIRE(ptr != nullptr, "lten_hip_fcq_forward_static: no device address for the static scratch");
		g_static_scratch[dev] = static_cast<unsigned char*>(ptr);  // zero-filled when the code object was loaded
	}
	unsigned char* base = g_static_scratch[dev];
	rs->split.partial = reinterpret_cast<int32_t*>(base);
	rs->split.partial_bytes = STATIC_SPLIT_BYTES;
	rs->terms = reinterpret_cast<int32_t*>(base + STATIC_SPLIT_BYTES);
	rs->terms_ints = STATIC_TERMS_INTS;
	rs->split.counters = reinterpret_cast<unsigned*>(base + STATIC_SPLIT_BYTES + STATIC_TERMS_INTS * 4);
	rs->split.max_tiles = STATIC_SPLIT_TILES;
	return 0;
}

// Called by lten_hip_init for the device it selects, so that the first lten_hip_fcq_forward_static on it (which may
// sit inside a recording) finds the address in place; the entry point still looks it up itself where init was skipped.
int prepare_static_scratch()
{
	RunScratch rs;
	return static_scratch(&rs);
}

}  // namespace lten_hip

using namespace lten_hip;

extern "C" {

int lten_hip_quantized_matmul(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, uint8_t alpha, const uint8_t* A,
                              const uint8_t* B, uint8_t beta, uint8_t* C, const lten_hip_qparams* qparams,
                              const int32_t* bias, int32_t* workspace)
{
	// l-ten/math_fns.cpp:1331-1334
	LTEN_HIP_REQUIRE(alpha == 1 && beta == 0, "Support for alpha != 1 and beta != 0 not implemented");
	return qgemm_run(tA, tB, M, N, K, A, B, C, 0, qparams, bias, workspace);
}

int lten_hip_quantized_matmul_acc(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, const uint8_t* A,
                                  const uint8_t* B, int32_t* acc, const lten_hip_qparams* qparams,
                                  const int32_t* bias, int32_t* workspace)
{
	return qgemm_run(tA, tB, M, N, K, A, B, acc, 1, qparams, bias, workspace);
}

int lten_hip_fcq_forward(uint64_t batch, uint64_t M, uint64_t in_features, uint64_t out_features, const uint8_t* X,
                         const uint8_t* W, const int32_t* bias, const lten_hip_qparams* qparams, uint8_t* Y,
                         int32_t* workspace)
{
	// l-ten/fully_connected.cpp:373-396 runs one quantized_matmul(false, true, M, out, in) per leading
	// index against the same weights.  Rows of the output are independent of each other, so the loop is
	// one GEMM with batch * M rows.
	return qgemm_run(0, 1, batch * M, out_features, in_features, X, W, Y, 0, qparams, bias, workspace);
}

int lten_hip_fcq_prepare_weights(const uint8_t* W, uint8_t* W_prepared, uint64_t out_features, uint64_t in_features, int32_t* weight_sums)
{
	const uint64_t count = out_features * in_features;
	if (count == 0) return 0;
	LTEN_HIP_REQUIRE(W && W_prepared, "lten_hip_fcq_prepare_weights: null pointer");
	LTEN_HIP_REQUIRE(((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(W_prepared)) & 15) == 0,
	                 "lten_hip_fcq_prepare_weights: both buffers must be 16-byte aligned");
	// rows of the prepared form start on 16-byte boundaries: in_features rounded up to a multiple of 16 bytes apart
	const uint64_t padded = (in_features + 15) & ~15ull;
	if (padded != in_features) {
		const uint8_t* w_end = W + count;
		const uint8_t* p_end = W_prepared + out_features * padded;
		LTEN_HIP_REQUIRE(w_end <= W_prepared || p_end <= W,
		                 "lten_hip_fcq_prepare_weights: in_features = %llu is no multiple of 16, so the prepared rows are padded to %llu bytes and "
		                 "the two buffers must not overlap", (unsigned long long)in_features, (unsigned long long)padded);
	}
	if (weight_sums != nullptr || padded != in_features) {
		LTEN_HIP_REQUIRE((reinterpret_cast<uintptr_t>(weight_sums) & 15) == 0, "lten_hip_fcq_prepare_weights: weight_sums must be 16-byte aligned");
		LTEN_HIP_REQUIRE(out_features < (1ull << 31) && in_features * 255ull < (1ull << 31), "lten_hip_fcq_prepare_weights: dimension too large");
		const unsigned blocks = (unsigned)ceil_div(out_features, 4);
		fcq_prepare_weights_sums_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(W, W_prepared, weight_sums, out_features, in_features, padded,
		                                                                           in_features % 16 == 0 ? 1 : 0);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	const uint64_t n16 = count / 16;
	const int tail = (int)(count % 16);
	const unsigned blocks = (unsigned)std::min<uint64_t>(std::max<uint64_t>(ceil_div(n16, 256), 1), 4096);
	fcq_prepare_weights_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(reinterpret_cast<const v4i*>(W), reinterpret_cast<v4i*>(W_prepared), n16,
	                                                                      W + n16 * 16, W_prepared + n16 * 16, tail);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int lten_hip_fcq_forward_prepared(uint64_t batch, uint64_t M, uint64_t in_features, uint64_t out_features, const uint8_t* X,
                                  const uint8_t* W_prepared, const int32_t* weight_sums, const int32_t* bias,
                                  const lten_hip_qparams* qparams, uint8_t* Y, int32_t* workspace)
{
	LTEN_HIP_REQUIRE(weight_sums != nullptr, "lten_hip_fcq_forward_prepared: weight_sums is null (lten_hip_fcq_prepare_weights fills it)");
	LTEN_HIP_REQUIRE((reinterpret_cast<uintptr_t>(weight_sums) & 15) == 0, "lten_hip_fcq_forward_prepared: weight_sums must be 16-byte aligned");
	return qgemm_run(0, 1, batch * M, out_features, in_features, X, W_prepared, Y, 0, qparams, bias, workspace, true, nullptr, weight_sums);
}

int lten_hip_fcq_forward_static(uint64_t batch, uint64_t M, uint64_t in_features, uint64_t out_features, const uint8_t* X,
                                const uint8_t* W, const int32_t* bias, const lten_hip_qparams* qparams, uint8_t* Y)
{
	LTEN_HIP_REQUIRE(batch * M + out_features <= STATIC_TERMS_INTS,
	                 "lten_hip_fcq_forward_static: batch * M + out_features = %llu exceeds the limit of %llu",
	                 (unsigned long long)(batch * M + out_features), (unsigned long long)STATIC_TERMS_INTS);
	RunScratch rs;
	if (int rc = static_scratch(&rs)) return rc;
	// The array keeps whatever the last call left.  The arrival counters of a split-K launch must start at zero, and
	// they do without a fill launch: the array is zero when the code object is loaded, and the workgroup that arrives
	// last at a tile stores zero into its counter again (qgemm_fast_kernel).
	LibraryScratchHold nothing_else(1ull << 60);  // no kernel choice below may reach for the library's growing block
	return qgemm_run(0, 1, batch * M, out_features, in_features, X, W, Y, 0, qparams, bias, nullptr, false, &rs);
}

}  // extern "C"
