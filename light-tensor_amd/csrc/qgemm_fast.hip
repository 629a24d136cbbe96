// Tuned int8 GEMM tiles for large NT problems (both operands contiguous in K, K a multiple of 16 and at least
// one k-step long, N a multiple of 4; M and N need not be multiples of the tile: a load that would start past
// the last row of an operand fetches the last row instead, and what is computed from it is not stored):
// BM x BN output tile (256 x 256, 256 x 128 or 128 x 128), k-steps of BK bytes, a ring of S LDS stages filled by direct global->LDS loads
// (no register staging), MFMA 32x32x32 int8.
//
// Data path per k-step: every wavefront issues its share of the stage's wave-wide 16-byte-per-lane
// loads; lane L of load q writes LDS slot q*64 + L of the stage, and the lane picks the *global* 16-byte
// chunk so that slot (row, physical chunk) holds logical chunk (physical ^ swz(row)) — the swizzled
// layout that keeps the later ds_read_b128 operand fetches free of bank conflicts, obtained here by
// permuting which lane fetches what.  Raw bytes land in LDS; the XOR with 0x80 that turns uint8 into the
// int8 the matrix cores multiply is applied to the operand registers after the ds_read — to the activations
// only when the weights were prepared (WPRE: B already holds int8, see lten_hip_fcq_prepare_weights).
//
// Pipeline: the k-step is cut into 32-byte k-slices.  While the MFMAs of one slice run, the operand
// registers of the next slice are read from LDS and sign-flipped (register double buffer).  One barrier
// per k-step, before its last slice: ahead of it a wavefront waits (vmcnt) for its own loads of stage
// kt+1; behind it every load of stage kt+1 has landed and every wavefront holds the last slice of stage kt
// in registers, so stage kt can be refilled with k-step kt+S.  The refill is spread over two beats (the one
// behind the barrier and the first of the next k-step, every other load each, one load per MFMA at most):
// all wavefronts of a CU issuing their whole share in one beat saturates the CU's memory pipeline for that
// beat and the wavefronts, which issue in order, stop feeding the matrix pipe while they queue.
//
// The zero-point terms of a tile (per row, per column, constant) are what its accumulators start from, so the
// epilogue is the requantize alone.  TERMS says where they come from: 0 = only the constant (both zero points 128, no
// bias); 1 = the vectors a launch of qgemm_terms_kernel left in the caller's workspace; 2 = the column term is worked
// out here from the weight sums kept since the weights were prepared (coef_b * wsum[n] + bias[n]) and there is no row
// term; 3 = the same, and the row term comes from the activation fragments on their way into the matrix cores: before
// the sign flip a fragment holds l-ten's uint8 bytes, and one instruction adds four of them to a sum.  The two wavefronts that multiply the same
// activation rows share that work (each sums the row blocks j with j % WN == wn), the sums meet in LDS behind the
// main loop and are added to the accumulators there.  No launch but this one runs in forms 2 and 3.
// The epilogue: a wavefront turns each of its 32-row blocks into bytes (the convert
// instruction drops its byte into the packed word itself), passes them through a strip of LDS of its own to
// get whole row segments of TN bytes, and stores those with the non-temporal hint (the output is not read
// again by this kernel, and lines that leave the L2 early do not have to be written back when the kernel ends).
#include "common.h"
#include "qgemm_common.h"
#include "lds_async.h"

namespace lten_hip {

template <int BM, int BN, int BK, int WM, int WN, int S, int OUT, int TERMS, bool SPLIT = false, bool TAIL = false, bool WPRE = false>
__global__ __launch_bounds__(WM* WN * 64) void qgemm_fast_kernel(QProblem p)
{
	constexpr int W = WM * WN;
	constexpr int CPR = BK / 16;           // 16-byte chunks per tile row
	constexpr int RPL = 64 / CPR;          // tile rows covered by one wave-wide load
	constexpr int NS = BK / 32;            // k-slices per k-step
	constexpr int STAGE = (BM + BN) * BK;  // bytes
	constexpr int LOADS = STAGE / 1024;    // wave-wide loads per stage
	constexpr int LPW = LOADS / W;         // per wavefront
	constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
	static_assert(LOADS % W == 0 && S >= 2 && S <= 4 && (S - 1) * LPW < 64 && NS >= 2 && NS % 2 == 0, "pipeline shape");

	constexpr int WP = TN + 16;  // row pitch of a wavefront's output strip in LDS (keeps rows 16-byte aligned)
	static_assert(W * 32 * WP <= S * STAGE, "the output strips fit into the operand stages");
	__shared__ __attribute__((aligned(1024))) uint8_t smem[S * STAGE];
	constexpr bool ROWSUM = TERMS == 3;
	// The accumulators of a requantizing launch run at a distance from zero (QProblem::acc_offset, added to what they
	// start from and taken off again before the convert; with wrapping int32 arithmetic the result is the same bit for
	// bit): sums that hover around zero change sign all the time, and every sign change toggles all upper bits of a
	// two's-complement accumulator in the matrix pipe, which costs clock under the part's power limit (4096^3 on
	// uniform x N(0,40) bytes: 56.9 -> 55.3 us on one part, the subtraction in the epilogue included).
	constexpr bool OFFSET = !SPLIT && OUT != Q_OUT_ACC;
	__shared__ int row_sums[ROWSUM ? BM : 1];  // TERMS == 3: byte sum over this workgroup's share of K, per tile row

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm = wave / WN, wn = wave % WN;

	// Workgroup -> tile.  Consecutive workgroup ids go round-robin to the 8 XCDs, each with its own L2;
	// every XCD gets one compact 4 x 8 block of tiles so that its CUs stream the same A and B rows.
	const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
	int tm, tn;
	{
		const int nb = tiles_m * tiles_n, bid = blockIdx.x;
		int lid = bid;
		if ((nb & 7) == 0) lid = (bid & 7) * (nb >> 3) + (bid >> 3);
		constexpr int GM = 4, GN = 8;
		if (tiles_m % GM == 0 && tiles_n % GN == 0) {
			const int group = lid / (GM * GN), within = lid % (GM * GN), groups_n = tiles_n / GN;
			tm = (group / groups_n) * GM + within / GN;
			tn = (group % groups_n) * GN + within % GN;
		} else {
			tm = lid / tiles_n;
			tn = lid % tiles_n;
		}
	}
	const int m0 = tm * BM, n0 = tn * BN;

	// ---- global -> LDS: what this lane fetches for each of its wavefront's loads.  Load q covers rows
	// q*RPL .. q*RPL+RPL-1 of the stacked [A tile; B tile]; wavefront w issues loads w, w+W, w+2W, ...,
	// so its first BM / RPL / W loads are A rows and the rest B rows whatever w is.
	static_assert((BM / RPL) % W == 0 && (BN / RPL) % W == 0 && LPW % 2 == 0, "A and B loads split evenly over the wavefronts and the two refill beats");
	constexpr int NA = BM / RPL / W;  // a wavefront's loads of A rows; the rest are B rows
	uint32_t voff[LPW];
	uint32_t lds_slot[LPW];
	bool in_tail[LPW];  // TAIL: this lane's chunk lies inside the last, partial k-step
	const uint32_t smem_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
#pragma unroll
	for (int i = 0; i < LPW; i++) {
		const int q = wave + i * W;
		const int r = q * RPL + lane / CPR;
		const int kc = (lane % CPR) ^ swz<CPR>(r);
		voff[i] = (i < NA ? (uint32_t)min(m0 + r, p.M - 1) : (uint32_t)min(n0 + r - BM, p.N - 1)) * (uint32_t)p.K + kc * 16;
		lds_slot[i] = smem_addr + q * 1024;
		in_tail[i] = kc * 16 < p.K % BK;
	}
	// with SPLIT, blockIdx.y picks this workgroup's share of K (whole k-steps; the first K / BK % splits shares are one step
	// longer than the rest); with TAIL the last k-step is partial (K % 16 == 0)
	const int share = SPLIT ? p.K / BK / p.splits : 0, longer = SPLIT ? p.K / BK - share * p.splits : 0;
	const int KT = SPLIT ? share + ((int)blockIdx.y < longer ? 1 : 0) : (TAIL ? (p.K + BK - 1) / BK : p.K / BK);
	const int64_t k_first = SPLIT ? ((int64_t)blockIdx.y * share + min((int)blockIdx.y, longer)) * BK : 0;
	const uint8_t* const a_base = p.A + k_first;
	const uint8_t* const b_base = p.B + k_first;
	// In the partial k-step a lane whose chunk lies past K loads nothing.  For the A tile it stores bytes of 0x80
	// instead, which the sign flip turns into zeros, so whatever the B tile still holds there is multiplied by 0.
	auto load_one = [&](int i, int stage, int kt) {
		if (TAIL && kt == KT - 1 && p.K % BK != 0) {
			if (in_tail[i]) {
				async_load16(lds_slot[i] + stage * STAGE, (i < NA ? a_base : b_base) + (int64_t)kt * BK, voff[i]);
			} else if (i < NA) {
				const v4i pad = { (int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080 };
				*reinterpret_cast<v4i*>(smem + (lds_slot[i] - smem_addr) + stage * STAGE + lane * 16) = pad;
			}
			return;
		}
		async_load16(lds_slot[i] + stage * STAGE, (i < NA ? a_base : b_base) + (int64_t)kt * BK, voff[i]);
	};
	auto issue = [&](int stage, int kt) {
#pragma unroll
		for (int i = 0; i < LPW; i++) load_one(i, stage, kt);
	};

	// ---- LDS -> MFMA operands.  Lane (lrow, lgrp) feeds row lrow of a 32-row block with the 16 bytes
	// lgrp of a 32-byte k-slice; slice s of the row sits at physical chunk (2s + lgrp) ^ swz(row).
	const int lrow = lane & 31, lgrp = lane >> 5;
	const int chunk0 = lgrp ^ swz<CPR>(lrow);
	const int off_w = BM * BK + (wn * TN + lrow) * BK + (chunk0 << 4);
	const int off_x = (wm * TM + lrow) * BK + (chunk0 << 4);
	// Which 32-row block of the wavefront's activation rows its fragment slot j holds: block j, except that with
	// TERMS == 3 and two wavefronts per row of wavefronts the second one holds them in the other order, so that "the
	// slot I sum" is slot 0 for both and the main loop needs no branch on the wavefront's number.
	static_assert(!ROWSUM || WN == 1 || (WN == 2 && FM == 2), "sharing of the row sums");
	const int jsw = (ROWSUM && WN == 2) ? wn : 0;
	int xblk[FM];  // byte offset of slot j's row block inside the activation tile
#pragma unroll
	for (int j = 0; j < FM; j++) xblk[j] = (j ^ jsw) * 32 * BK;

	// Accumulators start from the zero-point terms.  Lane (lrow, lgrp), register 4q + e of block (i, j) is the output at
	//   m = m0 + wm*TM + (j ^ jsw)*32 + lrow,  n = n0 + wn*TN + i*32 + 8q + 4*lgrp + e.
	// With SPLIT only the workgroup with the first share of K carries them.  The loads of the term vectors are issued
	// behind the first stages' loads (init_acc is called there): ahead of them they cost the prologue a second round
	// trip to memory, 2.5 us at 4096^3.
	v16i acc[FN][FM];
	auto init_acc = [&]() {
		const bool carry = !SPLIT || blockIdx.y == 0;
		int rt[FM];
#pragma unroll
		for (int j = 0; j < FM; j++) {
			rt[j] = carry ? p.konst : 0;
			if (OFFSET) rt[j] += p.acc_offset;
			if (TERMS == 1 && carry) rt[j] += p.rterm[min(m0 + wm * TM + (j ^ jsw) * 32 + lrow, p.M - 1)];
		}
		// Every load below is unconditional, from a column clamped into the matrix (with N % 4 == 0 four columns exist
		// together; what a clamped load brings is never stored), and the one choice, how the bias is fetched, is made
		// outside the loops: a branch per vector would make each load wait for the one before it.
		v4i ct[FN][4];
		const int ncol = n0 + wn * TN + lgrp * 4;
		const bool have = TERMS != 0 && carry;
#pragma unroll
		for (int i = 0; i < FN; i++)
#pragma unroll
			for (int q = 0; q < 4; q++) ct[i][q] = v4i{ 0, 0, 0, 0 };
		if ((p.N & 3) == 0) {
			if (TERMS == 1 && have) {
#pragma unroll
				for (int i = 0; i < FN; i++)
#pragma unroll
					for (int q = 0; q < 4; q++) ct[i][q] = *reinterpret_cast<const v4i*>(p.cterm + min(ncol + i * 32 + q * 8, p.N - 4));
			}
			if (TERMS >= 2 && have) {
#pragma unroll
				for (int i = 0; i < FN; i++)
#pragma unroll
					for (int q = 0; q < 4; q++) {
						const v4i ws = *reinterpret_cast<const v4i*>(p.wsum + min(ncol + i * 32 + q * 8, p.N - 4));
#pragma unroll
						for (int e = 0; e < 4; e++) ct[i][q][e] = ws[e] * p.coef_b;
					}
				if (p.bias != nullptr && (reinterpret_cast<uintptr_t>(p.bias) & 15) == 0) {
#pragma unroll
					for (int i = 0; i < FN; i++)
#pragma unroll
						for (int q = 0; q < 4; q++) ct[i][q] += *reinterpret_cast<const v4i*>(p.bias + min(ncol + i * 32 + q * 8, p.N - 4));
				} else if (p.bias != nullptr) {  // a bias vector that only has the alignment of its ints
#pragma unroll
					for (int i = 0; i < FN; i++)
#pragma unroll
						for (int q = 0; q < 4; q++) {
							const int32_t* b = p.bias + min(ncol + i * 32 + q * 8, p.N - 4);
							ct[i][q] += v4i{ b[0], b[1], b[2], b[3] };
						}
				}
			}
		} else if (have) {
			// N is no multiple of 4: the last columns do not come in fours, so every column is clamped and loaded by itself
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int q = 0; q < 4; q++)
#pragma unroll
					for (int e = 0; e < 4; e++) {
						const int col = min(ncol + i * 32 + q * 8 + e, p.N - 1);
						if (TERMS == 1) ct[i][q][e] = p.cterm[col];
						if (TERMS >= 2) ct[i][q][e] = p.wsum[col] * p.coef_b + (p.bias != nullptr ? p.bias[col] : 0);
					}
		}
#pragma unroll
		for (int i = 0; i < FN; i++)
#pragma unroll
			for (int q = 0; q < 4; q++)
#pragma unroll
				for (int j = 0; j < FM; j++)
#pragma unroll
					for (int e = 0; e < 4; e++) acc[i][j][q * 4 + e] = rt[j] + ct[i][q][e];
	};

	// TERMS == 3: this wavefront's share of the activation row sums, lane (lrow, lgrp) holding the bytes it has fed so
	// far.  A fragment is added up right before its sign flip, while it still holds l-ten's uint8 bytes: one
	// sum-of-absolute-differences against zero per dword (full rate; the 4 x int8 dot product that would take the
	// flipped bytes issues at a quarter of that and cost 3.2 us at 4096^3 against 0.9), each dword into a sum of its own
	// so that no instruction waits for the one before.
	constexpr int NSUM = WN == 1 ? FM : 1;  // row blocks (fragment slots) this wavefront sums
	unsigned rsum[NSUM][4];
#pragma unroll
	for (int j = 0; j < NSUM; j++)
#pragma unroll
		for (int d = 0; d < 4; d++) rsum[j][d] = 0;
	auto add_rowsum = [&](int j, const v4i& raw) {
		if (ROWSUM && j < NSUM) {
#pragma unroll
			for (int d = 0; d < 4; d++) rsum[j][d] = __builtin_amdgcn_sad_u8((unsigned)raw[d], 0u, rsum[j][d]);
		}
	};
	auto read_frags = [&](v4i(&fw)[FN], v4i(&fx)[FM], int stg, int s) {
		const uint8_t* sbase = smem + stg * STAGE;
#pragma unroll
		for (int i = 0; i < FN; i++) fw[i] = *reinterpret_cast<const v4i*>(sbase + (off_w ^ (s << 5)) + i * 32 * BK);
#pragma unroll
		for (int j = 0; j < FM; j++) fx[j] = *reinterpret_cast<const v4i*>(sbase + (off_x ^ (s << 5)) + xblk[j]);
	};
	auto flip_frags = [&](v4i(&fw)[FN], v4i(&fx)[FM]) {
		if (!WPRE) {
#pragma unroll
			for (int i = 0; i < FN; i++) fw[i] = flip_sign_bits(fw[i]);
		}
#pragma unroll
		for (int j = 0; j < FM; j++) {
			add_rowsum(j, fx[j]);
			fx[j] = flip_sign_bits(fx[j]);
		}
	};
	auto mma = [&](const v4i(&fw)[FN], const v4i(&fx)[FM]) {
#pragma unroll
		for (int i = 0; i < FN; i++)
#pragma unroll
			for (int j = 0; j < FM; j++)
				acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[i], fx[j], acc[i][j], 0, 0, 0);
	};
	// One pipeline beat in the exact instruction order wanted (scheduling fences keep the compiler from
	// regrouping it): the FM*FN MFMAs of the current slice, and in the shadow of each MFMA one piece of
	// the work for what comes next — first the LDS reads of the next slice's operands (one per MFMA), then
	// their sign flips, and, in the two beats that follow the barrier, this wavefront's refill loads: the
	// even-numbered ones in the first (refill == 1), the odd-numbered ones in the second (refill == 2), spaced
	// evenly over the beat's MFMAs.  Nothing is issued in a burst, so the matrix pipe never drains while the
	// wave is busy with address arithmetic or memory instructions.
	auto beat = [&](const v4i(&cw)[FN], const v4i(&cx)[FM], v4i(&nw)[FN], v4i(&nx)[FM], int stg, int s, int refill,
	                int refill_stage, int refill_kt) {
		constexpr int NR = FM + FN, NM = FM * FN;
		static_assert(NM >= NR, "one operand read and one flip per MFMA at most");
		constexpr int NFLIP = WPRE ? FM : NR;  // prepared weights: only the activations are flipped
		constexpr int FLIP0 = NM - NFLIP;      // flips ride on the last NFLIP MFMAs
		constexpr int HL = LPW / 2;            // refill loads per beat
		constexpr int STEP = NM >= HL ? NM / HL : 1;
		// A beat with as few MFMAs as operands (64 x 64 per wavefront: four and four) would flip each operand behind
		// the very MFMA that its read rode on, and wait out the LDS latency four times a beat: there the reads go
		// two at a time behind the first MFMAs (activations first) and all flips behind the last.
		constexpr bool DENSE = NM <= NR;
		const uint8_t* sbase = smem + stg * STAGE;
#pragma unroll
		for (int m = 0; m < NM; m++) {
			const int i = m / FM, j = m % FM;
			acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(cw[i], cx[j], acc[i][j], 0, 0, 0);
			if (DENSE) {
#pragma unroll
				for (int f = 2 * m; f < 2 * m + 2 && f < NR; f++) {
					if (f < FM) nx[f] = *reinterpret_cast<const v4i*>(sbase + (off_x ^ (s << 5)) + xblk[f]);
					else nw[f - FM] = *reinterpret_cast<const v4i*>(sbase + (off_w ^ (s << 5)) + (f - FM) * 32 * BK);
				}
				if (m == NM - 1) {
#pragma unroll
					for (int f = 0; f < FM; f++) {
						add_rowsum(f, nx[f]);
						nx[f] = flip_sign_bits(nx[f]);
					}
					if (!WPRE) {
#pragma unroll
						for (int f = 0; f < FN; f++) nw[f] = flip_sign_bits(nw[f]);
					}
				}
			} else {
				if (m < NR) {
					if (m < FN) nw[m] = *reinterpret_cast<const v4i*>(sbase + (off_w ^ (s << 5)) + m * 32 * BK);
					else nx[m - FN] = *reinterpret_cast<const v4i*>(sbase + (off_x ^ (s << 5)) + xblk[m - FN]);
				}
				if (m >= FLIP0) {
					const int f = m - FLIP0;
					if (WPRE) {
						add_rowsum(f, nx[f]);
						nx[f] = flip_sign_bits(nx[f]);
					} else if (f < FN) {
						nw[f] = flip_sign_bits(nw[f]);
					} else {
						add_rowsum(f - FN, nx[f - FN]);
						nx[f - FN] = flip_sign_bits(nx[f - FN]);
					}
				}
			}
			if (refill) {
#pragma unroll
				for (int h = 0; h < HL; h++)
					if ((h * STEP) % NM == m) load_one(2 * h + (refill - 1), refill_stage, refill_kt);
			}
			__builtin_amdgcn_sched_barrier(0);
		}
	};

	// Waits until at most n whole stages of this wavefront's loads (the youngest ones) are still in flight.  The count
	// holds only while every stage issues all LPW loads: with a partial last k-step in flight the caller asks for 0.
	auto wait_stages = [&](int n) {
		if (S >= 4 && n >= 2) wait_vmcnt<2 * LPW>();
		else if (S >= 3 && n == 1) wait_vmcnt<LPW>();
		else wait_vmcnt<0>();
	};
	v4i fw0[FN], fx0[FM], fw1[FN], fx1[FM];
	const int pre = min(S, KT);
	for (int st = 0; st < pre; st++) issue(st, st);
	init_acc();
	// with term vectors this wavefront's youngest loads are theirs, not a stage's: wait for everything
	if (TERMS != 0) wait_vmcnt<0>();
	else if (S == 2) { if (pre == 2) wait_vmcnt<LPW>(); else wait_vmcnt<0>(); }
	else wait_stages(TAIL && KT <= S ? 0 : pre - 1);
	__syncthreads();
	read_frags(fw0, fx0, 0, 0);
	flip_frags(fw0, fx0);

	// all slices of a k-step except the last: operands of slice s+1 come from the same stage; the first of
	// them carries the second half of the refill that the previous k-step's last beat began
	auto inner_beats = [&](int stg, int refill, int refill_stage, int refill_kt) {
#pragma unroll
		for (int s = 0; s + 1 < NS; s++) {
			const int rf = s == 0 ? refill : 0;
			if (s & 1) beat(fw1, fx1, fw0, fx0, stg, s + 1, rf, refill_stage, refill_kt);
			else beat(fw0, fx0, fw1, fx1, stg, s + 1, rf, refill_stage, refill_kt);
		}
	};

	int stage = 0, kt = 0;
	// steady state (branch-free apart from the first k-step's missing half refill): k-steps kt+1 .. kt+S-1 are in
	// flight or have landed (the youngest still lacks the second half of its loads), stage kt is refilled with
	// k-step kt+S once everybody has left it.  With S = 2 a load has one k-step of MFMAs to land, which covers the
	// memory latency when a CU holds two 128 x 128 tiles or one of 256 x 256; a CU with a single 128 x 128 tile
	// needs the deeper ring.
	for (; kt + S < KT; kt++) {
		const int next = stage + 1 == S ? 0 : stage + 1, prev = stage == 0 ? S - 1 : stage - 1;
		inner_beats(stage, kt > 0 ? 2 : 0, prev, kt + S - 1);
		wait_vmcnt<(S - 2) * LPW>();  // k-step kt+1 has landed
		__syncthreads();
		// NS is even: the last slice always sits in the second register set
		beat(fw1, fx1, fw0, fx0, next, 0, 1, stage, kt + S);
		stage = next;
	}
	// the second half of the last refill: in the first beat of the next k-step as before when there is one
	const bool half_open = kt > 0;
	// drain: nothing left to issue
	for (; kt < KT - 1; kt++) {
		const int next = stage + 1 == S ? 0 : stage + 1, prev = stage == 0 ? S - 1 : stage - 1;
		inner_beats(stage, (half_open && kt + S == KT) ? 2 : 0, prev, kt + S - 1);
		wait_stages(TAIL ? 0 : KT - kt - 2);
		__syncthreads();
		beat(fw1, fx1, fw0, fx0, next, 0, 0, 0, 0);
		stage = next;
	}
	inner_beats(stage, 0, 0, 0);
	mma(fw1, fx1);

	// TERMS == 3: the two k-halves of a row sit in lanes lrow and lrow + 32; the wavefront that summed row block j
	// leaves the sums in LDS, every wavefront of that row of wavefronts picks them up and adds coef_a times the sum to
	// the accumulators of the row (with SPLIT each workgroup adds its own share of K, which the exchange below sums).
	// The bytes that pad a partial last k-step are 0x80 before the flip and count 128 each: taken off again here.
	if (ROWSUM) {
#pragma unroll
		for (int j = 0; j < FM; j++)
			if (WN == 1 || j == 0) {
				const int mine = (int)(rsum[j < NSUM ? j : 0][0] + rsum[j < NSUM ? j : 0][1] + rsum[j < NSUM ? j : 0][2] + rsum[j < NSUM ? j : 0][3]);
				const int both = mine + __shfl_xor(mine, 32, 64) - (TAIL ? 128 * (KT * BK - p.K) : 0);
				if (lgrp == 0) row_sums[wm * TM + (j ^ jsw) * 32 + lrow] = both;
			}
		__syncthreads();
#pragma unroll
		for (int j = 0; j < FM; j++) {
			const int rt = row_sums[wm * TM + (j ^ jsw) * 32 + lrow] * p.coef_a - (OFFSET ? p.acc_offset : 0);
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int r = 0; r < 16; r++) acc[i][j][r] += rt;
		}
	}

	// Split K: every workgroup of a tile publishes its partial sums (in register order, so a wavefront of any of them
	// reads back exactly what the same wavefront of another wrote), then counts itself in; the one that arrives last
	// adds the others' sums to its own and carries on to the epilogue.  int32 sums do not depend on the order.  The
	// partial sums travel as device-scope atomic stores and loads (they pass the per-XCD L2s; plain stores behind a
	// release fence measured slower, because the fence writes back the whole L2), with a release fence before the count
	// and an acquire fence after it; nobody waits for anybody.  The last workgroup resets the counter for the next
	// launch on the stream.
	if (SPLIT) {
		constexpr int NACC = FN * FM * 16;
		int32_t* const tile_slabs = p.split_partial + (int64_t)blockIdx.x * p.splits * (NACC * W * 64);
		int32_t* const mine = tile_slabs + (int64_t)blockIdx.y * (NACC * W * 64);
#pragma unroll
		for (int i = 0; i < FN; i++)
#pragma unroll
			for (int j = 0; j < FM; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					__hip_atomic_store(mine + ((i * FM + j) * 16 + r) * (W * 64) + tid, acc[i][j][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
		__syncthreads();
		unsigned* const arrived = reinterpret_cast<unsigned*>(smem);  // the operand stages are no longer read
		if (tid == 0) *arrived = __hip_atomic_fetch_add(p.split_counters + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__syncthreads();
		if (*arrived != (unsigned)p.splits - 1) return;
		__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
		for (int s2 = 0; s2 < p.splits; s2++) {
			if (s2 == (int)blockIdx.y) continue;
			const int32_t* other = tile_slabs + (int64_t)s2 * (NACC * W * 64);
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int j = 0; j < FM; j++)
#pragma unroll
					for (int r = 0; r < 16; r++)
						acc[i][j][r] += __hip_atomic_load(other + ((i * FM + j) * 16 + r) * (W * 64) + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		}
		if (tid == 0) __hip_atomic_store(p.split_counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}

	if (OUT == Q_OUT_ACC) {
#pragma unroll
		for (int j = 0; j < FM; j++) {
			const int m = m0 + wm * TM + (j ^ jsw) * 32 + lrow;
			if (m >= p.M) continue;
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int q = 0; q < 4; q++) {
					const int n = n0 + wn * TN + i * 32 + q * 8 + lgrp * 4;
					if (n >= p.N) continue;
					if ((p.N & 3) == 0) {  // the four columns exist together, on a 16-byte boundary
						const v4i v = { acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3] };
						*reinterpret_cast<v4i*>(static_cast<int*>(p.C) + (int64_t)m * p.N + n) = v;
					} else {
#pragma unroll
						for (int e = 0; e < 4; e++)
							if (n + e < p.N) static_cast<int*>(p.C)[(int64_t)m * p.N + n + e] = acc[i][j][q * 4 + e];
					}
				}
		}
	} else {
		// The accumulator layout gives every lane 4 consecutive bytes of 32 different rows, which as direct stores would
		// be 8-byte fragments scattered over 32 cache lines per instruction.  Each wavefront therefore passes its 32 x TN
		// blocks through a strip of LDS of its own (no workgroup barrier beyond the one that retires the operand
		// stages), reads them back 16 bytes per lane and stores whole row segments; the stores of one block overlap the
		// arithmetic of the next.
		__syncthreads();  // every wavefront is done reading operand stages (SPLIT: and the arrival word)
		uint8_t* const strip = smem + wave * (32 * WP);
		const int epi_off = (OFFSET && !ROWSUM) ? p.acc_offset : 0;  // with row sums the offset went out with the row term
		const int row0 = m0 + wm * TM, col0 = n0 + wn * TN;
		uint8_t* const cbase = static_cast<uint8_t*>(p.C) + (int64_t)row0 * p.N + col0;
#pragma unroll
		for (int j = 0; j < FM; j++) {
			const int jrow = (j ^ jsw) * 32;  // the tile rows of this slot
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int q = 0; q < 4; q++) {
					unsigned word = 0;
					if (OUT == Q_OUT_U8_FAST) {
						requant_into<0>(word, acc[i][j][q * 4 + 0] - epi_off, p.mult, p.zp_c);
						requant_into<1>(word, acc[i][j][q * 4 + 1] - epi_off, p.mult, p.zp_c);
						requant_into<2>(word, acc[i][j][q * 4 + 2] - epi_off, p.mult, p.zp_c);
						requant_into<3>(word, acc[i][j][q * 4 + 3] - epi_off, p.mult, p.zp_c);
					} else {
						const unsigned b0 = requant<OUT>(acc[i][j][q * 4] - epi_off, p.mult, p.zp_c), b1 = requant<OUT>(acc[i][j][q * 4 + 1] - epi_off, p.mult, p.zp_c);
						const unsigned b2 = requant<OUT>(acc[i][j][q * 4 + 2] - epi_off, p.mult, p.zp_c), b3 = requant<OUT>(acc[i][j][q * 4 + 3] - epi_off, p.mult, p.zp_c);
						word = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
					}
					*reinterpret_cast<unsigned*>(strip + lrow * WP + i * 32 + q * 8 + lgrp * 4) = word;
				}
			wait_vmcnt_lgkm0<63>();  // this wavefront's strip is written
			__builtin_amdgcn_wave_barrier();
			if ((p.N & 15) == 0) {  // rows of C start on 16-byte boundaries: whole 16-byte pieces
				constexpr int LPS = TN / 16;   // lanes per row segment
				constexpr int RPI = 64 / LPS;  // rows per store instruction
#pragma unroll
				for (int t = 0; t < 32 / RPI; t++) {
					const int r = t * RPI + lane / LPS, ch = lane % LPS;
					const v4i val = *reinterpret_cast<const v4i*>(strip + r * WP + ch * 16);
					if (row0 + jrow + r < p.M && col0 + ch * 16 < p.N)
						__builtin_nontemporal_store(val, reinterpret_cast<v4i*>(cbase + (int64_t)(jrow + r) * p.N + ch * 16));
				}
			} else if ((p.N & 3) == 0) {  // four bytes at a time
				for (int c = lane; c < 32 * (TN / 4); c += 64) {
					const int r = c / (TN / 4), dw = c % (TN / 4);
					if (row0 + jrow + r < p.M && col0 + dw * 4 < p.N)
						*reinterpret_cast<int*>(cbase + (int64_t)(jrow + r) * p.N + dw * 4) = *reinterpret_cast<const int*>(strip + r * WP + dw * 4);
				}
			} else {
				// Rows of C start on any byte.  A row's piece of the strip is stored as the aligned dwords of C that lie inside
				// it (each put together from the two strip dwords that hold its bytes), then the up to three bytes before the
				// first and after the last of them, two lanes a row.  (Byte by byte it is 64 store instructions a block
				// instead of 21, and every one of them costs the memory pipeline the same: 4 us more at 300 x 1001 x 512.)
				const int cols = min(TN, p.N - col0);  // bytes of a row's piece that exist
				constexpr int SLOTS = TN / 4 + 1;
				for (int c = lane; c < 32 * SLOTS; c += 64) {
					const int r = c / SLOTS, d = c - r * SLOTS;
					uint8_t* const rowp = cbase + (int64_t)(jrow + r) * p.N;
					const int s = 4 * d - (int)(reinterpret_cast<uintptr_t>(rowp) & 3);  // first byte of the slot within the piece
					if (row0 + jrow + r < p.M && s >= 0 && s + 4 <= cols) {
						const int at = r * WP + s;
						const uint32_t* al = reinterpret_cast<const uint32_t*>(strip + (at & ~3));
						const uint32_t lo = al[0], hi = al[(at & 3) ? 1 : 0];
						*reinterpret_cast<uint32_t*>(rowp + s) = __builtin_amdgcn_alignbyte(hi, lo, (unsigned)(at & 3));
					}
				}
				{
					const int r = lane >> 1;
					uint8_t* const rowp = cbase + (int64_t)(jrow + r) * p.N;
					const int a = (int)(reinterpret_cast<uintptr_t>(rowp) & 3);
					const int head = min((4 - a) & 3, cols);             // bytes before the first aligned dword
					const int full = (cols - head) & ~3;                 // bytes stored as dwords above
					const int from = (lane & 1) ? head + full : 0, to = (lane & 1) ? cols : head;
					if (row0 + jrow + r < p.M) {
#pragma unroll
						for (int e = 0; e < 3; e++)
							if (from + e < to) rowp[from + e] = strip[r * WP + from + e];
					}
				}
			}
			wait_vmcnt_lgkm0<63>();  // the strip is read before the next block overwrites it
			__builtin_amdgcn_wave_barrier();
		}
	}
}

// Which TERMS form a launch takes; -1 = a combination these kernels are not built for (prepared weights with the
// vectors of qgemm_terms_kernel, raw weights with kept sums): the caller falls back to the general kernels.
static int fast_terms_mode(const QProblem& p)
{
	const bool wpre = p.b_flip == 0;
	if (p.wsum != nullptr) return wpre && p.rterm == nullptr && p.cterm == nullptr ? (p.coef_a != 0 ? 3 : 2) : -1;
	if (p.rterm != nullptr) return wpre ? -1 : 1;
	return 0;
}

// How far from zero a requantizing launch keeps its accumulators (see OFFSET in the kernel): the smallest of
// 0x2AAAAAAA, 0x0AAAAAAA, 0x02AAAAAA, ... that no sum of K products of two int8 values can bring below zero.  The
// alternating bits keep the distance clear of a power of two, where a sum that passes it would toggle a run of bits
// just as a change of sign does (4096^3: 0x800000 55.5 us, 0xAAAAAA 54.9, 0x2AAAAAAA 55.1, none 56.4).
static int32_t accumulator_offset(int K)
{
	int32_t off = 0x2AAAAAAA;
	while ((off >> 2) >= (int64_t)K * 16384) off >>= 2;
	return off;
}

// The reported kernel name says which zero-point terms the launch worked out itself.
static void set_fast_name(const char* name, int terms)
{
	char full[96];
	snprintf(full, sizeof(full), "%s%s", name, terms == 3 ? "+zpcol+zprow" : terms == 2 ? "+zpcol" : "");
	set_kernel_name(full);
}

template <int BM, int BN, int BK, int WM, int WN, int S, bool TAIL = false, bool WPRE = false>
static int launch_fast(const QProblem& q, int out, const char* name)
{
	if (!TAIL && q.K % BK != 0) return -1;
	QProblem p = q;
	p.acc_offset = accumulator_offset(p.K);
	const dim3 grid((unsigned)(ceil_div(p.M, BM) * ceil_div(p.N, BN))), block(WM * WN * 64);
	// prepared weights come with their sums (TERMS 2 or 3, or 0 when no term is needed), raw weights with the vectors of
	// qgemm_terms_kernel (1 or 0): see fast_terms_mode
	const int terms = fast_terms_mode(p);
	if (terms < 0) return -1;
	set_fast_name(name, terms);
#define LTEN_LAUNCH(OUTV)                                                                                            \
	if (WPRE && terms == 3)                                                                                      \
		qgemm_fast_kernel<BM, BN, BK, WM, WN, S, OUTV, WPRE ? 3 : 0, false, TAIL, WPRE><<<grid, block, 0, stream()>>>(p); \
	else if (WPRE && terms == 2)                                                                                 \
		qgemm_fast_kernel<BM, BN, BK, WM, WN, S, OUTV, WPRE ? 2 : 0, false, TAIL, WPRE><<<grid, block, 0, stream()>>>(p); \
	else if (!WPRE && terms == 1)                                                                                \
		qgemm_fast_kernel<BM, BN, BK, WM, WN, S, OUTV, WPRE ? 0 : 1, false, TAIL, WPRE><<<grid, block, 0, stream()>>>(p); \
	else                                                                                                         \
		qgemm_fast_kernel<BM, BN, BK, WM, WN, S, OUTV, 0, false, TAIL, WPRE><<<grid, block, 0, stream()>>>(p);
	if (out == Q_OUT_U8_FAST) { LTEN_LAUNCH(Q_OUT_U8_FAST) }
	else if (out == Q_OUT_U8_EXACT) { LTEN_LAUNCH(Q_OUT_U8_EXACT) }
	else { LTEN_LAUNCH(Q_OUT_ACC) }
#undef LTEN_LAUNCH
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// Scratch of the split-K launches: owned by the library, allocated on first use (never while a launch graph is
// being recorded), kept until the process ends.  One stream uses it at a time, as everything else in this library.
static SplitScratch g_split = { nullptr, 32u << 20, nullptr, 4096 };

static bool split_scratch_ready()
{
	if (g_split.partial != nullptr) return true;
	if (capturing()) return false;
	void* partial = nullptr;
	void* counters = nullptr;
	if (hipMalloc(&partial, g_split.partial_bytes) != hipSuccess) { (void)hipGetLastError(); return false; }
	if (hipMalloc(&counters, g_split.max_tiles * sizeof(unsigned)) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(partial); return false; }
	if (hipMemset(counters, 0, g_split.max_tiles * sizeof(unsigned)) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(partial); (void)hipFree(counters); return false; }
	g_split.partial = static_cast<int32_t*>(partial);
	g_split.counters = static_cast<unsigned*>(counters);
	return true;
}

// 128 x 128 tiles with K cut into `splits` shares; -1 when the problem or the scratch does not allow it.
int qgemm_fast_split_dispatch(const QProblem& q, int out, int splits, const SplitScratch* scratch)
{
	constexpr int T = 128, BK = 128;
	QProblem p = q;
	if (scratch == nullptr) {
		if (!split_scratch_ready()) return -1;
		scratch = &g_split;
	}
	const uint64_t tiles = ceil_div(p.M, T) * ceil_div(p.N, T);
	const bool fits = p.a_ks == 1 && p.b_ks == 1 && p.vec_ok && p.K % BK == 0 &&
	                  p.K / BK / splits >= 2 && splits >= 2 && splits <= 16 &&
	                  (uint64_t)p.M * p.K < (1ull << 32) && (uint64_t)p.N * p.K < (1ull << 32) &&
	                  (reinterpret_cast<uintptr_t>(p.C) & 15) == 0 && (p.cterm == nullptr || (reinterpret_cast<uintptr_t>(p.cterm) & 15) == 0) &&
	                  (reinterpret_cast<uintptr_t>(p.wsum) & 15) == 0 &&
	                  tiles * T * T * 4 * splits <= scratch->partial_bytes && tiles <= (uint64_t)scratch->max_tiles;
	if (!fits) return -1;
	p.split_partial = scratch->partial;
	p.split_counters = scratch->counters;
	p.splits = splits;
	const dim3 grid((unsigned)tiles, (unsigned)splits), block(256);
	const int terms = fast_terms_mode(p);
	if (terms < 0) return -1;
	const bool wpre = p.b_flip == 0;
	// a ring of four stages where a CU holds one workgroup anyway and the share of K is long enough to repay the
	// longer prologue (see launch_tile128)
	const bool deep = p.K / splits >= 4096 && tiles * splits <= 256;
	set_fast_name(deep ? (wpre ? "qgemm_fast_128x128x128_w2x2_s4_splitk_wpre" : "qgemm_fast_128x128x128_w2x2_s4_splitk")
	                   : (wpre ? "qgemm_fast_128x128x128_w2x2_s2_splitk_wpre" : "qgemm_fast_128x128x128_w2x2_s2_splitk"), terms);
#define LTEN_LAUNCH3(OUTV, TERMSV, WPREV)                                                                           \
	if (deep) qgemm_fast_kernel<T, T, BK, 2, 2, 4, OUTV, TERMSV, true, false, WPREV><<<grid, block, 0, stream()>>>(p); \
	else qgemm_fast_kernel<T, T, BK, 2, 2, 2, OUTV, TERMSV, true, false, WPREV><<<grid, block, 0, stream()>>>(p);
#define LTEN_LAUNCH(OUTV)                                                     \
	if (terms == 3) { LTEN_LAUNCH3(OUTV, 3, true) }                           \
	else if (terms == 2) { LTEN_LAUNCH3(OUTV, 2, true) }                      \
	else if (terms == 1) { LTEN_LAUNCH3(OUTV, 1, false) }                     \
	else if (wpre) { LTEN_LAUNCH3(OUTV, 0, true) }                            \
	else { LTEN_LAUNCH3(OUTV, 0, false) }
	if (out == Q_OUT_U8_FAST) { LTEN_LAUNCH(Q_OUT_U8_FAST) }
	else if (out == Q_OUT_U8_EXACT) { LTEN_LAUNCH(Q_OUT_U8_EXACT) }
	else { LTEN_LAUNCH(Q_OUT_ACC) }
#undef LTEN_LAUNCH
#undef LTEN_LAUNCH3
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// 128 x 128 tiles for outputs too small to give every CU a 256 x 256 tile.  Two stages let a CU hold two workgroups,
// whose MFMAs cover each other's load latency; where there is at most one workgroup per CU anyway, a ring of four
// stages does that, once K is long enough to repay the longer prologue (4096 x 4096 weights at M = 512: 21.6 -> 17.4
// us, 8192 x 8192 at M = 256: 41.4 -> 30.8 us; 2048 x 2048 at M = 512: 10.0 -> 10.7 us, so not there).
static int launch_tile128(const QProblem& p, int out, bool ktail, bool wpre)
{
	const bool deep = p.K >= 4096 && ceil_div(p.M, 128) * ceil_div(p.N, 128) <= 256;
	if (deep) {
		if (wpre) return ktail ? launch_fast<128, 128, 128, 2, 2, 4, true, true>(p, out, "qgemm_fast_128x128x128_w2x2_s4_ktail_wpre")
		                       : launch_fast<128, 128, 128, 2, 2, 4, false, true>(p, out, "qgemm_fast_128x128x128_w2x2_s4_wpre");
		return ktail ? launch_fast<128, 128, 128, 2, 2, 4, true>(p, out, "qgemm_fast_128x128x128_w2x2_s4_ktail")
		             : launch_fast<128, 128, 128, 2, 2, 4>(p, out, "qgemm_fast_128x128x128_w2x2_s4");
	}
	if (wpre) return ktail ? launch_fast<128, 128, 128, 2, 2, 2, true, true>(p, out, "qgemm_fast_128x128x128_w2x2_s2_ktail_wpre")
	                       : launch_fast<128, 128, 128, 2, 2, 2, false, true>(p, out, "qgemm_fast_128x128x128_w2x2_s2_wpre");
	return ktail ? launch_fast<128, 128, 128, 2, 2, 2, true>(p, out, "qgemm_fast_128x128x128_w2x2_s2_ktail")
	             : launch_fast<128, 128, 128, 2, 2, 2>(p, out, "qgemm_fast_128x128x128_w2x2_s2");
}

int qgemm_fast_dispatch(const QProblem& p, int out, int variant)
{
	// preconditions of the direct-to-LDS tiles; the caller falls back to the general kernels otherwise
	// K: any multiple of 16 from 32 on (variants 33, 41 and 51; a K below the k-step is one partial step), or a multiple of the k-step
	const bool fits = p.a_ks == 1 && p.b_ks == 1 && p.vec_ok && p.K % 16 == 0 && p.K >= 32 &&
	                  (uint64_t)p.M * p.K < (1ull << 32) && (uint64_t)p.N * p.K < (1ull << 32) &&
	                  (reinterpret_cast<uintptr_t>(p.C) & 15) == 0 &&
	                  (p.cterm == nullptr || (reinterpret_cast<uintptr_t>(p.cterm) & 15) == 0) &&
	                  (reinterpret_cast<uintptr_t>(p.wsum) & 15) == 0;
	if (!fits) return -1;
	const bool wpre = p.b_flip == 0;
	const bool ktail = p.K % 128 != 0;
	switch (variant) {
	// 256 x 256 tiles: eight wavefronts of 64 x 128 (the activation operand is the one with fewer fragments
	// per wavefront, so prepared weights leave two fragments per k-slice to flip)
	case 33:
		if (wpre) return ktail ? launch_fast<256, 256, 128, 4, 2, 2, true, true>(p, out, "qgemm_fast_256x256x128_w4x2_s2_ktail_wpre")
		                       : launch_fast<256, 256, 128, 4, 2, 2, false, true>(p, out, "qgemm_fast_256x256x128_w4x2_s2_wpre");
		return ktail ? launch_fast<256, 256, 128, 4, 2, 2, true>(p, out, "qgemm_fast_256x256x128_w4x2_s2_ktail")
		             : launch_fast<256, 256, 128, 4, 2, 2>(p, out, "qgemm_fast_256x256x128_w4x2_s2");
	// the same tile with the wavefronts laid out the other way round (raw weights only)
	case 34: return wpre ? -1 : launch_fast<256, 256, 128, 2, 4, 2>(p, out, "qgemm_fast_256x256x128_w2x4_s2");
	// 128 x 128 tiles for outputs too small to give every CU a 256 x 256 tile
	case 41: return launch_tile128(p, out, ktail, wpre);
	// 256 x 128 tiles, four wavefronts of 64 x 128, three stages (144 KB): for outputs that give every CU about one such
	// tile and too few 256 x 256 ones; a k-step brings 48 KB through the CU's vector L1 for 1024 clocks of MFMAs where
	// two 128 x 128 tiles bring 64 KB (2048 x 4096 x 4096: 36.1 -> 32.8 us)
	case 51:
		if (wpre) return ktail ? launch_fast<256, 128, 128, 4, 1, 3, true, true>(p, out, "qgemm_fast_256x128x128_w4x1_s3_ktail_wpre")
		                       : launch_fast<256, 128, 128, 4, 1, 3, false, true>(p, out, "qgemm_fast_256x128x128_w4x1_s3_wpre");
		return ktail ? launch_fast<256, 128, 128, 4, 1, 3, true>(p, out, "qgemm_fast_256x128x128_w4x1_s3_ktail")
		             : launch_fast<256, 128, 128, 4, 1, 3>(p, out, "qgemm_fast_256x128x128_w4x1_s3");
	default: return -1;
	}
}

}  // namespace lten_hip
