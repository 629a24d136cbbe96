// fp32 GEMM tiles for large problems with 16-byte-aligned operand rows, in all four layouts: T x T output tile (256 or 128), k-steps of
// 32, a ring of S LDS stages filled by direct global->LDS loads (no register staging), MFMA 32x32x2 fp32.
//
// An operand tile is staged the way it lies in memory:
//   contiguous in k (A not transposed, B transposed): [tile row][32 k] = 128-byte rows of eight 16-byte
//     chunks; the lane that loads a chunk is chosen so that row r holds logical chunk c at position
//     c ^ swz(r), which keeps the 16-byte operand reads free of bank conflicts;
//   contiguous along the tile row (A transposed, B not transposed): [32 k][T rows], read one float per lane.
// A k-step is cut into four slices of 8 k.  In a slice lane (lrow, lk) feeds tile row lrow of a 32-row block with
// k = 8s + 4lk + t for the t-th of four MFMAs; the assignment is the same for A and B, which is all a dot
// product needs.  While the MFMAs of one slice run, the operands of the next are read from LDS (register
// double buffer), one read in the shadow of each MFMA.  One barrier per k-step, before its last slice: ahead of
// it a wavefront waits (vmcnt) for its own loads of stage kt+1; behind it every load of stage kt+1 has landed and
// every wavefront holds the last slice of stage kt in registers, so stage kt is refilled at once with k-step kt+S.
//
// MFMA rows are rows of op(A), columns are columns of op(B): a lane holds one output column n and 16 rows,
// so that a store instruction writes two full 128-byte rows of C.
//
// M and N need not be multiples of the tile: a load that would start past the last row of an operand starts at
// the last one instead (a row that exists, fetched twice), and the outputs computed from it are not stored.
#include "common.h"
#include "gemm_f32_core.h"
#include "lds_async.h"
#include "qgemm_common.h"
#include "sgemm_common.h"

namespace lten_hip {

template <int T, int WM, int WN, int S, bool A_KC, bool B_KC>
__global__ __launch_bounds__(WM* WN * 64) void sgemm_fast_kernel(SProblem p)
{
	constexpr int BK = 32;                     // floats per k-step
	constexpr int W = WM * WN;
	constexpr int NS = 4;                      // slices of 8 k
	constexpr int TILE = T * BK * 4;           // bytes of one operand tile
	constexpr int STAGE = 2 * TILE;
	constexpr int LOADS = STAGE / 1024, LPW = LOADS / W;
	constexpr int TM = T / WM, TN = T / WN, FM = TM / 32, FN = TN / 32;
	constexpr int RA = A_KC ? FM : 4 * FM, RB = B_KC ? FN : 4 * FN;  // LDS reads per slice
	constexpr int NR = RA + RB, NM = FM * FN * 4;
	static_assert(LOADS % W == 0 && LPW % 2 == 0 && (T / 8) % W == 0, "A and B loads split evenly over the wavefronts");
	static_assert(S >= 2 && S <= 4 && (S - 2) * LPW < 64 && 2 * NM >= NR && NM >= LPW, "pipeline shape");
	__shared__ __attribute__((aligned(1024))) uint8_t smem[S * STAGE];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm = wave / WN, wn = wave % WN;
	const int lrow = lane & 31, lk = lane >> 5;

	// Workgroup -> tile.  Consecutive workgroup ids go round-robin to the 8 XCDs, each with its own L2; every
	// XCD gets compact 4 x 8 blocks of tiles so that its CUs stream the same rows of A and B.
	// A batch of small problems (problems_by_xcd): XCD x takes problems x, x + 8, ... whole, so that a problem's operands
	// cross one L2 only (the workgroups of the grid go round-robin to the XCDs in the order z * gridDim.x + x).
	const int tiles_m = (p.M + T - 1) / T, tiles_n = (p.N + T - 1) / T;
	int tm, tn, bz = blockIdx.z;
	{
		const int nb = tiles_m * tiles_n, bid = blockIdx.x;
		int lid = bid;
		if (p.problems_by_xcd) {
			const unsigned linear = blockIdx.z * (unsigned)nb + bid, j = linear >> 3;
			const unsigned prob = j / (unsigned)nb;  // (the division runs on the vector ALU: back to scalar registers)
			bz = __builtin_amdgcn_readfirstlane((int)prob * 8 + (int)(linear & 7));
			lid = __builtin_amdgcn_readfirstlane((int)(j - prob * (unsigned)nb));
		} else if ((nb & 7) == 0) lid = (bid & 7) * (nb >> 3) + (bid >> 3);
		constexpr int GM = 4, GN = 8;
		if (tiles_m % GM == 0 && tiles_n % GN == 0) {
			const int group = lid / (GM * GN), within = lid % (GM * GN), groups_n = tiles_n / GN;
			tm = (group / groups_n) * GM + within / GN;
			tn = (group % groups_n) * GN + within % GN;
		} else if (tiles_m < tiles_n && (nb & 7) == 0 && !p.problems_by_xcd) {
			// a wide product (few rows of tiles; tiles in a multiple of 8, so an XCD has a run of them): the run walks down the
			// columns of tiles, so that the XCD reads a narrow range of B and all of the smaller A (256 x 6272 x 2304, 4 x 98
			// tiles: B crossed the L2s 3.4 times with the run along a row of tiles)
			tn = lid / tiles_m;
			tm = lid % tiles_m;
		} else {
			tm = lid / tiles_n;
			tn = lid % tiles_n;
		}
	}
	const int m0 = tm * T, n0 = tn * T;
	const float* A = p.A + (int64_t)bz * p.stride_a;
	const float* B = p.B + (int64_t)bz * p.stride_b;
	float* C = p.C + (int64_t)bz * p.stride_c;

	// ---- global -> LDS.  Load q (1 KB) of a tile: k-contiguous: rows 8q .. 8q+7, lane -> (row 8q + L/8, chunk
	// (L%8) ^ swz(row)); row-contiguous: k rows (1024 / (4T)) q .., lane -> 4 consecutive tile rows of one k.
	// Wavefront w issues loads w, w+W, ...: its first LPW/2 are A, the rest B.
	uint32_t voff[LPW], lds_slot[LPW];
	const uint32_t smem_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
#pragma unroll
	for (int i = 0; i < LPW; i++) {
		const bool is_a = i < LPW / 2;
		const int q = wave + (is_a ? i : i - LPW / 2) * W;
		const bool kc_layout = is_a ? A_KC : B_KC;
		const uint32_t ld = (uint32_t)(is_a ? p.lda : p.ldb);
		const int row0 = is_a ? m0 : n0, rows = is_a ? p.M : p.N;
		if (kc_layout) {
			const int r = q * 8 + (lane >> 3);
			const int c = (lane & 7) ^ swz<8>(r);
			voff[i] = ((uint32_t)min(row0 + r, rows - 1) * ld + c * 4) * 4;
		} else {
			constexpr int KPL = 256 / T, LPR = T / 4;  // k rows per load, lanes per k row
			const int k = q * KPL + lane / LPR, r4 = (lane % LPR) * 4;
			// (rows is a multiple of 4, or the caller has promised that the array's rows can be read up to the next one)
			voff[i] = (k * ld + (uint32_t)min(row0 + r4, ((rows + 3) & ~3) - 4)) * 4;
		}
		lds_slot[i] = smem_addr + (is_a ? 0 : TILE) + q * 1024;
	}
	const int64_t a_step = A_KC ? BK : (int64_t)BK * p.lda, b_step = B_KC ? BK : (int64_t)BK * p.ldb;
	auto load_one = [&](int i, int stage, int kt) {
		const float* base = i < LPW / 2 ? A + kt * a_step : B + kt * b_step;
		async_load16(lds_slot[i] + stage * STAGE, base, voff[i]);
	};
	auto issue = [&](int stage, int kt) {
#pragma unroll
		for (int i = 0; i < LPW; i++) load_one(i, stage, kt);
	};

	// ---- LDS -> MFMA operands
	const int chunk0 = lk ^ swz<8>(lrow);
	const int off_a = A_KC ? (wm * TM + lrow) * 128 + (chunk0 << 4) : (4 * lk * T + wm * TM + lrow) * 4;
	const int off_b = TILE + (B_KC ? (wn * TN + lrow) * 128 + (chunk0 << 4) : (4 * lk * T + wn * TN + lrow) * 4);
	// read number e of slice s (operands of one slice: fa[FM][4], fb[FN][4])
	auto read_one = [&](float (&fa)[FM][4], float (&fb)[FN][4], const uint8_t* sbase, int s, int e) {
		if (e < RA) {
			if (A_KC) {
				const float4 v = *reinterpret_cast<const float4*>(sbase + (off_a ^ (s << 5)) + e * 32 * 128);
				fa[e][0] = v.x; fa[e][1] = v.y; fa[e][2] = v.z; fa[e][3] = v.w;
			} else {
				fa[e >> 2][e & 3] = *reinterpret_cast<const float*>(sbase + off_a + ((8 * s + (e & 3)) * T + (e >> 2) * 32) * 4);
			}
		} else {
			const int f = e - RA;
			if (B_KC) {
				const float4 v = *reinterpret_cast<const float4*>(sbase + (off_b ^ (s << 5)) + f * 32 * 128);
				fb[f][0] = v.x; fb[f][1] = v.y; fb[f][2] = v.z; fb[f][3] = v.w;
			} else {
				fb[f >> 2][f & 3] = *reinterpret_cast<const float*>(sbase + off_b + ((8 * s + (f & 3)) * T + (f >> 2) * 32) * 4);
			}
		}
	};

	v16f acc[FM][FN];
#pragma unroll
	for (int i = 0; i < FM; i++)
#pragma unroll
		for (int j = 0; j < FN; j++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

	const int KT = p.K / BK;

	// One pipeline beat in the exact instruction order wanted (scheduling fences keep the compiler from
	// regrouping it): the MFMAs of the current slice and, in the shadow of each, one LDS read of the next slice's
	// operands and, in the beat that follows the barrier, this wavefront's refill loads.
	auto beat = [&](const float (&ca)[FM][4], const float (&cb)[FN][4], float (&na)[FM][4], float (&nb)[FN][4], int stg, int s,
	                bool read_next, bool refill, int refill_stage, int refill_kt) {
		const uint8_t* sbase = smem + stg * STAGE;
#pragma unroll
		for (int m = 0; m < NM; m++) {
			const int t = m / (FM * FN), blk = m % (FM * FN), i = blk / FN, j = blk % FN;  // neighbours use different accumulators
			acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[i][t], cb[j][t], acc[i][j], 0, 0, 0);
			if (read_next) {  // one operand read behind each MFMA; two where a 32 x 32 wavefront tile has fewer MFMAs per slice than reads
#pragma unroll
				for (int e = m; e < NR; e += NM) read_one(na, nb, sbase, s, e);
			}
			if (refill) {
#pragma unroll
				for (int l = m; l < LPW; l += NM) load_one(l, refill_stage, refill_kt);
			}
			__builtin_amdgcn_sched_barrier(0);
		}
	};
	auto wait_steps = [&](int steps) {
		if (steps >= 2 && S >= 4) wait_vmcnt<(S >= 4 ? 2 : 0) * LPW>();
		else if (steps >= 1 && S >= 3) wait_vmcnt<(S >= 3 ? 1 : 0) * LPW>();
		else wait_vmcnt<0>();
	};

	float fa0[FM][4], fb0[FN][4], fa1[FM][4], fb1[FN][4];
	const int pre = min(S, KT);
	for (int st = 0; st < pre; st++) issue(st, st);
	wait_steps(pre - 1);
	__syncthreads();
#pragma unroll
	for (int e = 0; e < NR; e++) read_one(fa0, fb0, smem, 0, e);

	// slices 0 .. NS-2 of a k-step: the operands of slice s+1 come from the same stage
	auto inner_beats = [&](int stg) {
#pragma unroll
		for (int s = 0; s + 1 < NS; s++) {
			if (s & 1) beat(fa1, fb1, fa0, fb0, stg, s + 1, true, false, 0, 0);
			else beat(fa0, fb0, fa1, fb1, stg, s + 1, true, false, 0, 0);
		}
	};

	int stage = 0, kt = 0;
	// steady state (branch-free): k-steps kt+2 .. kt+S-1 are in flight behind stage kt+1
	for (; kt + S < KT; kt++) {
		inner_beats(stage);
		wait_vmcnt_lgkm0<(S - 2) * LPW>();  // own loads of stage kt+1 landed, own reads of stage kt done
		__syncthreads();
		const int next = (stage + 1 == S) ? 0 : stage + 1;
		beat(fa1, fb1, fa0, fb0, next, 0, true, true, stage, kt + S);  // NS is even: the last slice sits in set 1
		stage = next;
	}
	// drain: nothing left to issue, fewer loads in flight
	for (; kt < KT - 1; kt++) {
		inner_beats(stage);
		wait_steps(min(S - 2, KT - 2 - kt));
		wait_vmcnt_lgkm0<63>();
		__syncthreads();
		const int next = (stage + 1 == S) ? 0 : stage + 1;
		beat(fa1, fb1, fa0, fb0, next, 0, true, false, 0, 0);
		stage = next;
	}
	inner_beats(stage);
	beat(fa1, fb1, fa0, fb0, stage, 0, false, false, 0, 0);

	// Epilogue: register 4q + e of block (i, j) of lane (lrow, lk) is
	//   m = m0 + wm*TM + 32i + 8q + 4lk + e,  n = n0 + wn*TN + 32j + lrow.
	// The address is a part the wavefront shares plus a lane offset.
	float bv[FN];
#pragma unroll
	for (int j = 0; j < FN; j++) {
		const int n = n0 + wn * TN + j * 32 + lrow;
		bv[j] = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
	}
	if (p.col_group != 0) {  // grouped columns (alpha = 1, beta = 0, a bias per row): the lane's columns are placed one by one
		int64_t coff[FN];
#pragma unroll
		for (int j = 0; j < FN; j++) {
			const unsigned n = (unsigned)(n0 + wn * TN + j * 32 + lrow), grp = n / (unsigned)p.col_group;
			coff[j] = n < (unsigned)p.N ? (int64_t)grp * p.col_group_stride + (n - grp * (unsigned)p.col_group) : -1;
		}
#pragma unroll
		for (int i = 0; i < FM; i++)
#pragma unroll
			for (int r = 0; r < 16; r++) {
				const int m = m0 + wm * TM + i * 32 + (r >> 2) * 8 + 4 * lk + (r & 3);
				if (m >= p.M) continue;
				float* cr = C + (int64_t)m * p.ldc;
				const float rb = p.row_bias ? p.row_bias[m] : 0.0f;
#pragma unroll
				for (int j = 0; j < FN; j++)
					if (coff[j] >= 0) cr[coff[j]] = acc[i][j][r] + rb;
			}
		return;
	}
	float* cw = C + (int64_t)(m0 + wm * TM) * p.ldc + n0 + wn * TN;
	const unsigned c_lane = (unsigned)(4 * lk * p.ldc) + lrow;
	if (m0 + T <= p.M && n0 + T <= p.N) {
#pragma unroll
		for (int i = 0; i < FM; i++)
#pragma unroll
			for (int r = 0; r < 16; r++) {
				float* cr = cw + (int64_t)(i * 32 + (r >> 2) * 8 + (r & 3)) * p.ldc;
#pragma unroll
				for (int j = 0; j < FN; j++) {
					float v = p.alpha * acc[i][j][r];
					if (p.beta != 0.0f) v += p.beta * cr[c_lane + j * 32];
					__builtin_nontemporal_store(v + bv[j], &cr[c_lane + j * 32]);  // C is written once and not read again here
				}
			}
		return;
	}
#pragma unroll
	for (int i = 0; i < FM; i++)
#pragma unroll
		for (int r = 0; r < 16; r++) {
			if (m0 + wm * TM + i * 32 + (r >> 2) * 8 + 4 * lk + (r & 3) >= p.M) continue;
			float* cr = cw + (int64_t)(i * 32 + (r >> 2) * 8 + (r & 3)) * p.ldc;
#pragma unroll
			for (int j = 0; j < FN; j++) {
				if (n0 + wn * TN + j * 32 + lrow >= p.N) continue;
				float v = p.alpha * acc[i][j][r];
				if (p.beta != 0.0f) v += p.beta * cr[c_lane + j * 32];
				cr[c_lane + j * 32] = v + bv[j];
			}
		}
}

template <int T, int WM, int WN, int S>
static int launch_fast(const SProblem& q, int tA, int tB, uint64_t batch, const char* name)
{
	SProblem p = q;
	const uint64_t nb = ceil_div(p.M, T) * ceil_div(p.N, T);
	// (problems of at most 64 tiles, a whole number of them per XCD; larger ones spread over the XCDs in compact blocks)
	p.problems_by_xcd = batch >= 8 && batch % 8 == 0 && nb <= 64 && nb * batch < (1ull << 31) ? 1 : 0;
	const dim3 grid((unsigned)nb, 1, (unsigned)batch), block(WM * WN * 64);
	set_kernel_name(name);
	if (!tA && !tB) sgemm_fast_kernel<T, WM, WN, S, true, false><<<grid, block, 0, stream()>>>(p);
	if (!tA && tB) sgemm_fast_kernel<T, WM, WN, S, true, true><<<grid, block, 0, stream()>>>(p);
	if (tA && !tB) sgemm_fast_kernel<T, WM, WN, S, false, false><<<grid, block, 0, stream()>>>(p);
	if (tA && tB) sgemm_fast_kernel<T, WM, WN, S, false, true><<<grid, block, 0, stream()>>>(p);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int sgemm_fast_dispatch(const SProblem& p, int tA, int tB, uint64_t batch, int variant)
{
	// preconditions of the direct-to-LDS tiles; the caller falls back to the general kernels otherwise
	const uint64_t a_rows = tA ? p.K : p.M, b_rows = tB ? p.N : p.K;  // rows of the arrays as stored
	// an operand that is contiguous along its tile rows is fetched four rows at a time: whole groups of four only
	const bool slack = rows_readable_to_pitch();
	const bool fits = (!tA || p.M % 4 == 0 || (slack && (uint64_t)p.lda >= (((uint64_t)p.M + 3) & ~3ull))) &&
	                  (tB || p.N % 4 == 0 || (slack && (uint64_t)p.ldb >= (((uint64_t)p.N + 3) & ~3ull))) && p.M >= 4 && p.N >= 4 &&
	                  p.K % 32 == 0 && p.K >= 64 && (p.lda & 3) == 0 && (p.ldb & 3) == 0 &&
	                  (p.stride_a & 3) == 0 && (p.stride_b & 3) == 0 &&
	                  ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0 &&
	                  a_rows * (uint64_t)p.lda < (1ull << 30) && b_rows * (uint64_t)p.ldb < (1ull << 30) &&  // 32-bit byte offsets
	                  4ull * (uint64_t)p.ldc + 32 < (1ull << 32) && p.rowsum == nullptr;
	if (!fits) return -1;
	switch (variant) {
	case 11: return launch_fast<256, 2, 4, 2>(p, tA, tB, batch, "sgemm_fast_256x256x32_w2x4_s2");
	case 12: return launch_fast<256, 4, 2, 2>(p, tA, tB, batch, "sgemm_fast_256x256x32_w4x2_s2");
	case 21: return launch_fast<128, 2, 2, 2>(p, tA, tB, batch, "sgemm_fast_128x128x32_w2x2_s2");
	case 22: return launch_fast<128, 2, 2, 3>(p, tA, tB, batch, "sgemm_fast_128x128x32_w2x2_s3");
	case 23: return launch_fast<128, 2, 2, 4>(p, tA, tB, batch, "sgemm_fast_128x128x32_w2x2_s4");
	// 64 x 64 tiles (a 32 x 32 tile per wavefront): up to two operand reads ride behind an MFMA when an operand is
	// row-contiguous
	case 31: return launch_fast<64, 2, 2, 2>(p, tA, tB, batch, "sgemm_fast_64x64x32_w2x2_s2");
	default: return -1;
	}
}

}  // namespace lten_hip
