// Tuned int8 GEMM tiles for large NT problems (both operands contiguous in K, K a multiple of the
// k-step or, for two of the tiles, of 16; N a multiple of 4; M and N need not be multiples of the tile: a load that would start past the
// last row of an operand fetches the last row instead, and what is computed from it is not stored):
// 256 x 256 output tile, k-steps of BK bytes, a ring of S LDS stages filled by
// direct global->LDS loads (no register staging), MFMA 32x32x32 int8.
//
// Data path per k-step: every wavefront issues its share of the stage's wave-wide 16-byte-per-lane
// loads; lane L of load q writes LDS slot q*64 + L of the stage, and the lane picks the *global* 16-byte
// chunk so that slot (row, physical chunk) holds logical chunk (physical ^ swz(row)) — the swizzled
// layout that keeps the later ds_read_b128 operand fetches free of bank conflicts, obtained here by
// permuting which lane fetches what.  Raw bytes land in LDS; the XOR with 0x80 that turns uint8 into the
// int8 the matrix cores multiply is applied to the operand registers after the ds_read.
//
// Pipeline: the k-step is cut into 32-byte k-slices.  While the MFMAs of one slice run, the operand
// registers of the next slice are read from LDS and sign-flipped (register double buffer).  One barrier
// per k-step, before its last slice: ahead of it a wavefront waits (vmcnt) for its own loads of stage
// kt+1; behind it every load of stage kt+1 has landed and every wavefront holds the last slice of stage kt
// in registers, so stage kt is refilled at once with k-step kt+S.
//
// Epilogue: zero-point terms, requantize, then the bytes are staged through LDS so that global memory is
// written in whole 256-byte rows.
#include "common.h"
#include "qgemm_common.h"
#include "lds_async.h"

namespace lten_hip {

// Phase timestamps for tuning builds (-DLTEN_HIP_STAMPS): slots 0..3 = start, main loop start, main loop
// end, end in the 100 MHz wall clock; slots 4..5 = start / main loop end in shader clocks.
#ifdef LTEN_HIP_STAMPS
#define LTEN_STAMP(slot)                                                                                              \
	do {                                                                                                          \
		if (threadIdx.x == 0 && p.stamps) p.stamps[blockIdx.x * 8 + (slot)] = (slot) < 4 ? wall_clock64() : clock64(); \
	} while (0)
#else
#define LTEN_STAMP(slot) do { } while (0)
#endif
// Tuning builds may switch pieces of the main loop off (results are then wrong; timing only):
// bit 0 no refill loads, bit 1 no sign flips, bit 2 no LDS operand reads, bit 3 no barrier.
#ifndef LTEN_HIP_EXP
#define LTEN_HIP_EXP 0
#endif

template <int T, int BK, int WM, int WN, int S, int OUT, bool TERMS, bool SPLIT = false, bool TAIL = false>
__global__ __launch_bounds__(WM* WN * 64) void qgemm_fast_kernel(QProblem p)
{
	constexpr int BM = T, BN = T;  // square output tile, 256 or 128
	constexpr int W = WM * WN;
	constexpr int CPR = BK / 16;           // 16-byte chunks per tile row
	constexpr int RPL = 64 / CPR;          // tile rows covered by one wave-wide load
	constexpr int NS = BK / 32;            // k-slices per k-step
	constexpr int STAGE = (BM + BN) * BK;  // bytes
	constexpr int LOADS = STAGE / 1024;    // wave-wide loads per stage
	constexpr int LPW = LOADS / W;         // per wavefront
	constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
	static_assert(LOADS % W == 0 && S >= 2 && S <= 4 && (S - 2) * LPW < 64 && NS % 2 == 0, "pipeline shape");

	constexpr int OLD = BN + 16;  // row pitch of the output tile staged in LDS by the epilogue
	constexpr int LDS_BYTES = S * STAGE > BM * OLD ? S * STAGE : BM * OLD;
	__shared__ __attribute__((aligned(1024))) uint8_t smem[LDS_BYTES];

	LTEN_STAMP(0);
	LTEN_STAMP(4);
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
	// so its first LPW/2 loads are A rows and the rest B rows whatever w is.
	static_assert((BM / RPL) % W == 0 && LPW % 2 == 0, "A and B loads split evenly over the wavefronts");
	uint32_t voff[LPW];
	uint32_t lds_slot[LPW];
	bool in_tail[LPW];  // TAIL: this lane's chunk lies inside the last, partial k-step
	const uint32_t smem_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
#pragma unroll
	for (int i = 0; i < LPW; i++) {
		const int q = wave + i * W;
		const int r = q * RPL + lane / CPR;
		const int kc = (lane % CPR) ^ swz<CPR>(r);
		voff[i] = (i < LPW / 2 ? (uint32_t)min(m0 + r, p.M - 1) : (uint32_t)min(n0 + r - BM, p.N - 1)) * (uint32_t)p.K + kc * 16;
		lds_slot[i] = smem_addr + q * 1024;
		in_tail[i] = kc * 16 < p.K % BK;
	}
	// with SPLIT, blockIdx.y picks this workgroup's share of K; with TAIL the last k-step is partial (K % 16 == 0)
	const int KT = SPLIT ? p.K / BK / p.splits : (TAIL ? (p.K + BK - 1) / BK : p.K / BK);
	const uint8_t* const a_base = p.A + (SPLIT ? (int64_t)blockIdx.y * KT * BK : 0);
	const uint8_t* const b_base = p.B + (SPLIT ? (int64_t)blockIdx.y * KT * BK : 0);
	// In the partial k-step a lane whose chunk lies past K loads nothing.  For the A tile it stores bytes of 0x80
	// instead, which the sign flip turns into zeros, so whatever the B tile still holds there is multiplied by 0.
	auto load_one = [&](int i, int stage, int kt) {
		if (TAIL && kt == KT - 1 && p.K % BK != 0) {
			if (in_tail[i]) {
				async_load16(lds_slot[i] + stage * STAGE, (i < LPW / 2 ? a_base : b_base) + (int64_t)kt * BK, voff[i]);
			} else if (i < LPW / 2) {
				const v4i pad = { (int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080 };
				*reinterpret_cast<v4i*>(smem + (lds_slot[i] - smem_addr) + stage * STAGE + lane * 16) = pad;
			}
			return;
		}
		async_load16(lds_slot[i] + stage * STAGE, (i < LPW / 2 ? a_base : b_base) + (int64_t)kt * BK, voff[i]);
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

	v16i acc[FN][FM];
#pragma unroll
	for (int i = 0; i < FN; i++)
#pragma unroll
		for (int j = 0; j < FM; j++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

	auto read_frags = [&](v4i(&fw)[FN], v4i(&fx)[FM], int stg, int s) {
		const uint8_t* sbase = smem + stg * STAGE;
#pragma unroll
		for (int i = 0; i < FN; i++) fw[i] = *reinterpret_cast<const v4i*>(sbase + (off_w ^ (s << 5)) + i * 32 * BK);
#pragma unroll
		for (int j = 0; j < FM; j++) fx[j] = *reinterpret_cast<const v4i*>(sbase + (off_x ^ (s << 5)) + j * 32 * BK);
	};
	auto flip_frags = [&](v4i(&fw)[FN], v4i(&fx)[FM]) {
#pragma unroll
		for (int i = 0; i < FN; i++) fw[i] = flip_sign_bits(fw[i]);
#pragma unroll
		for (int j = 0; j < FM; j++) fx[j] = flip_sign_bits(fx[j]);
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
	// their sign flips, and, in the beat that follows the barrier, this wavefront's refill loads (one per
	// MFMA).  Nothing is issued in a burst, so the matrix pipe never drains while the wave is busy with
	// address arithmetic or memory instructions.
	auto beat = [&](const v4i(&cw)[FN], const v4i(&cx)[FM], v4i(&nw)[FN], v4i(&nx)[FM], int stg, int s, bool refill,
	                int refill_stage, int refill_kt) {
		constexpr int NR = FM + FN, NM = FM * FN;
		static_assert(NM >= NR, "one operand read and one flip per MFMA at most");
		constexpr int FLIP0 = NM - NR;  // flips ride on the last NR MFMAs
		const uint8_t* sbase = smem + stg * STAGE;
#pragma unroll
		for (int m = 0; m < NM; m++) {
			const int i = m / FM, j = m % FM;
			acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(cw[i], cx[j], acc[i][j], 0, 0, 0);
			if (m < NR && !(LTEN_HIP_EXP & 4)) {
				if (m < FN) nw[m] = *reinterpret_cast<const v4i*>(sbase + (off_w ^ (s << 5)) + m * 32 * BK);
				else nx[m - FN] = *reinterpret_cast<const v4i*>(sbase + (off_x ^ (s << 5)) + (m - FN) * 32 * BK);
			}
			if (m >= FLIP0 && !(LTEN_HIP_EXP & 2)) {
				const int f = m - FLIP0;
				if (f < FN) nw[f] = flip_sign_bits(nw[f]);
				else nx[f - FN] = flip_sign_bits(nx[f - FN]);
			}
			if (refill && !(LTEN_HIP_EXP & 1)) {
#pragma unroll
				for (int l = m; l < LPW; l += NM) load_one(l, refill_stage, refill_kt);
			}
			__builtin_amdgcn_sched_barrier(0);
		}
	};
	// waits until at most `steps` k-steps' worth of this wavefront's loads are still in flight
	auto wait_steps = [&](int steps) {
		if (steps >= 2 && S >= 4) wait_vmcnt<(S >= 4 ? 2 : 0) * LPW>();
		else if (steps >= 1 && S >= 3) wait_vmcnt<(S >= 3 ? 1 : 0) * LPW>();
		else wait_vmcnt<0>();
	};

	v4i fw0[FN], fx0[FM], fw1[FN], fx1[FM];
	const int pre = min(S, KT);
	for (int st = 0; st < pre; st++) issue(st, st);
	wait_steps(pre - 1);
	__syncthreads();
	read_frags(fw0, fx0, 0, 0);
	flip_frags(fw0, fx0);
	LTEN_STAMP(1);

	// all slices of a k-step except the last: operands of slice s+1 come from the same stage
	auto inner_beats = [&](int stg) {
#pragma unroll
		for (int s = 0; s + 1 < NS; s++) {
			if (s & 1) beat(fw1, fx1, fw0, fx0, stg, s + 1, false, 0, 0);
			else beat(fw0, fx0, fw1, fx1, stg, s + 1, false, 0, 0);
		}
	};

	int stage = 0, kt = 0;
	// steady state (branch-free): k-steps kt+2 .. kt+S-1 are in flight behind stage kt+1
	for (; kt + S < KT; kt++) {
		inner_beats(stage);
		wait_vmcnt<(S - 2) * LPW>();
		if (!(LTEN_HIP_EXP & 8)) __syncthreads();
		const int next = (stage + 1 == S) ? 0 : stage + 1;
		// NS is even: the last slice always sits in the second register set
		beat(fw1, fx1, fw0, fx0, next, 0, true, stage, kt + S);
		stage = next;
	}
	// drain: nothing left to issue, fewer loads in flight
	for (; kt < KT - 1; kt++) {
		inner_beats(stage);
		wait_steps(min(S - 2, KT - 2 - kt));
		__syncthreads();
		const int next = (stage + 1 == S) ? 0 : stage + 1;
		beat(fw1, fx1, fw0, fx0, next, 0, false, 0, 0);
		stage = next;
	}
	inner_beats(stage);
	mma(fw1, fx1);
	LTEN_STAMP(2);
	LTEN_STAMP(5);

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

	// Epilogue: lane (lrow, lgrp), register 4q + e of block (i, j) is the output at
	//   m = m0 + wm*TM + j*32 + lrow,  n = n0 + wn*TN + i*32 + 8q + 4*lgrp + e.
	if (OUT == Q_OUT_ACC) {
#pragma unroll
		for (int j = 0; j < FM; j++) {
			const int m = m0 + wm * TM + j * 32 + lrow;
			if (m >= p.M) continue;
			const int rt = TERMS ? p.rterm[m] + p.konst : p.konst;
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int q = 0; q < 4; q++) {
					const int n = n0 + wn * TN + i * 32 + q * 8 + lgrp * 4;
					if (n >= p.N) continue;  // N is a multiple of 4: the four columns exist together
					v4i v = { acc[i][j][q * 4] + rt, acc[i][j][q * 4 + 1] + rt, acc[i][j][q * 4 + 2] + rt, acc[i][j][q * 4 + 3] + rt };
					if (TERMS) v += *reinterpret_cast<const v4i*>(p.cterm + n);
					*reinterpret_cast<v4i*>(static_cast<int*>(p.C) + (int64_t)m * p.N + n) = v;
				}
		}
	} else {
		// Requantized bytes go through LDS so that global memory sees whole rows: the accumulator layout
		// gives every lane 4 consecutive bytes of 32 different rows, which as direct stores would be 8-byte
		// fragments scattered over 32 cache lines per instruction.  The tile is staged as [256][256 + 16]
		// bytes (the pad keeps rows 16-byte aligned and spreads the 4-byte writes over the banks), then
		// copied out 16 bytes per lane, 4 full 256-byte rows per wave-wide store.
		__syncthreads();  // every wavefront is done reading operand stages
#pragma unroll
		for (int j = 0; j < FM; j++) {
			const int row = wm * TM + j * 32 + lrow;
			const int rt = TERMS ? p.rterm[min(m0 + row, p.M - 1)] + p.konst : p.konst;
#pragma unroll
			for (int i = 0; i < FN; i++)
#pragma unroll
				for (int q = 0; q < 4; q++) {
					const int col = wn * TN + i * 32 + q * 8 + lgrp * 4;
					int v[4];
#pragma unroll
					for (int e = 0; e < 4; e++) v[e] = acc[i][j][q * 4 + e] + rt;
					if (TERMS && n0 + col < p.N) {
						const v4i ct = *reinterpret_cast<const v4i*>(p.cterm + n0 + col);
						v[0] += ct.x; v[1] += ct.y; v[2] += ct.z; v[3] += ct.w;
					}
					const unsigned b0 = requant<OUT>(v[0], p.mult, p.zp_c), b1 = requant<OUT>(v[1], p.mult, p.zp_c);
					const unsigned b2 = requant<OUT>(v[2], p.mult, p.zp_c), b3 = requant<OUT>(v[3], p.mult, p.zp_c);
					*reinterpret_cast<unsigned*>(smem + row * OLD + col) = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
				}
		}
		__syncthreads();
		uint8_t* cout = static_cast<uint8_t*>(p.C) + (int64_t)m0 * p.N + n0;
		if ((p.N & 15) == 0) {  // rows of C start on 16-byte boundaries: whole 16-byte pieces
#pragma unroll
			for (int c = tid; c < BM * BN / 16; c += W * 64) {
				const int row = c / (BN / 16), ch = c % (BN / 16);
				if (m0 + row < p.M && n0 + ch * 16 < p.N)
					*reinterpret_cast<v4i*>(cout + (int64_t)row * p.N + ch * 16) = *reinterpret_cast<const v4i*>(smem + row * OLD + ch * 16);
			}
		} else {  // N is a multiple of 4: four bytes at a time
			for (int c = tid; c < BM * BN / 4; c += W * 64) {
				const int row = c / (BN / 4), dw = c % (BN / 4);
				if (m0 + row < p.M && n0 + dw * 4 < p.N)
					*reinterpret_cast<int*>(cout + (int64_t)row * p.N + dw * 4) = *reinterpret_cast<const int*>(smem + row * OLD + dw * 4);
			}
		}
	}
#ifdef LTEN_HIP_STAMPS
	__syncthreads();
	LTEN_STAMP(3);
#endif
}

template <int T, int BK, int WM, int WN, int S, bool TAIL = false>
static int launch_fast(const QProblem& p, int out, const char* name)
{
	if (!TAIL && p.K % BK != 0) return -1;
	const dim3 grid((unsigned)(ceil_div(p.M, T) * ceil_div(p.N, T))), block(WM * WN * 64);
	const bool terms = p.rterm != nullptr;
	set_kernel_name(name);
#define LTEN_LAUNCH(OUTV)                                                                                      \
	if (terms)                                                                                             \
		qgemm_fast_kernel<T, BK, WM, WN, S, OUTV, true, false, TAIL><<<grid, block, 0, stream()>>>(p);      \
	else                                                                                                   \
		qgemm_fast_kernel<T, BK, WM, WN, S, OUTV, false, false, TAIL><<<grid, block, 0, stream()>>>(p);
	if (out == Q_OUT_U8_FAST) { LTEN_LAUNCH(Q_OUT_U8_FAST) }
	else if (out == Q_OUT_U8_EXACT) { LTEN_LAUNCH(Q_OUT_U8_EXACT) }
	else { LTEN_LAUNCH(Q_OUT_ACC) }
#undef LTEN_LAUNCH
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// Scratch of the split-K launches: owned by the library, allocated on first use (never while a launch graph is
// being recorded), kept until the process ends.  One stream uses it at a time, as everything else in this library.
static int32_t* g_split_partial = nullptr;
static unsigned* g_split_counters = nullptr;
constexpr size_t SPLIT_PARTIAL_BYTES = 32u << 20;
constexpr int SPLIT_MAX_TILES = 4096;

static bool split_scratch_ready()
{
	if (g_split_partial != nullptr) return true;
	if (capturing()) return false;
	void* partial = nullptr;
	void* counters = nullptr;
	if (hipMalloc(&partial, SPLIT_PARTIAL_BYTES) != hipSuccess) { (void)hipGetLastError(); return false; }
	if (hipMalloc(&counters, SPLIT_MAX_TILES * sizeof(unsigned)) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(partial); return false; }
	if (hipMemset(counters, 0, SPLIT_MAX_TILES * sizeof(unsigned)) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(partial); (void)hipFree(counters); return false; }
	g_split_partial = static_cast<int32_t*>(partial);
	g_split_counters = static_cast<unsigned*>(counters);
	return true;
}

// 128 x 128 tiles with K cut into `splits` shares; -1 when the problem or the scratch does not allow it.
int qgemm_fast_split_dispatch(const QProblem& q, int out, int splits)
{
	constexpr int T = 128, BK = 128;
	QProblem p = q;
	const bool fits = p.a_ks == 1 && p.b_ks == 1 && p.vec_ok && p.N % 4 == 0 && p.K % (BK * splits) == 0 &&
	                  p.K / splits >= 2 * BK && splits >= 2 && splits <= 16 &&
	                  (uint64_t)p.M * p.K < (1ull << 32) && (uint64_t)p.N * p.K < (1ull << 32) &&
	                  (reinterpret_cast<uintptr_t>(p.C) & 15) == 0 && (p.cterm == nullptr || (reinterpret_cast<uintptr_t>(p.cterm) & 15) == 0) &&
	                  ceil_div(p.M, T) * ceil_div(p.N, T) * T * T * 4 * splits <= SPLIT_PARTIAL_BYTES && ceil_div(p.M, T) * ceil_div(p.N, T) <= SPLIT_MAX_TILES;
	if (!fits || !split_scratch_ready()) return -1;
	p.split_partial = g_split_partial;
	p.split_counters = g_split_counters;
	p.splits = splits;
	const dim3 grid((unsigned)(ceil_div(p.M, T) * ceil_div(p.N, T)), (unsigned)splits), block(256);
	const bool terms = p.rterm != nullptr;
	set_kernel_name("qgemm_fast_128x128x128_w2x2_s2_splitk");
#define LTEN_LAUNCH(OUTV)                                                                              \
	if (terms)                                                                                     \
		qgemm_fast_kernel<T, BK, 2, 2, 2, OUTV, true, true><<<grid, block, 0, stream()>>>(p);       \
	else                                                                                           \
		qgemm_fast_kernel<T, BK, 2, 2, 2, OUTV, false, true><<<grid, block, 0, stream()>>>(p);
	if (out == Q_OUT_U8_FAST) { LTEN_LAUNCH(Q_OUT_U8_FAST) }
	else if (out == Q_OUT_U8_EXACT) { LTEN_LAUNCH(Q_OUT_U8_EXACT) }
	else { LTEN_LAUNCH(Q_OUT_ACC) }
#undef LTEN_LAUNCH
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int qgemm_fast_dispatch(const QProblem& p, int out, int variant)
{
	// preconditions of the direct-to-LDS tiles; the caller falls back to the general kernels otherwise
	// K: a multiple of the k-step, or (variants 33 and 41) any multiple of 16 at least one k-step long
	const bool fits = p.a_ks == 1 && p.b_ks == 1 && p.vec_ok && p.N % 4 == 0 && p.K % 16 == 0 && p.K >= 128 &&
	                  (uint64_t)p.M * p.K < (1ull << 32) && (uint64_t)p.N * p.K < (1ull << 32) &&
	                  (reinterpret_cast<uintptr_t>(p.C) & 15) == 0 &&
	                  (p.cterm == nullptr || (reinterpret_cast<uintptr_t>(p.cterm) & 15) == 0);
	if (!fits) return -1;
	switch (variant) {
	case 21: return launch_fast<256, 64, 2, 2, 3>(p, out, "qgemm_fast_256x256x64_w2x2_s3");
	case 23: return launch_fast<256, 64, 2, 4, 3>(p, out, "qgemm_fast_256x256x64_w2x4_s3");
	case 24: return launch_fast<256, 64, 4, 2, 3>(p, out, "qgemm_fast_256x256x64_w4x2_s3");
	case 26: return launch_fast<256, 64, 4, 2, 4>(p, out, "qgemm_fast_256x256x64_w4x2_s4");
	case 28: return launch_fast<256, 64, 4, 2, 2>(p, out, "qgemm_fast_256x256x64_w4x2_s2");
	case 31: return launch_fast<256, 128, 2, 2, 2>(p, out, "qgemm_fast_256x256x128_w2x2_s2");
	case 33:
		if (p.K % 128 != 0) return launch_fast<256, 128, 2, 4, 2, true>(p, out, "qgemm_fast_256x256x128_w2x4_s2_ktail");
		return launch_fast<256, 128, 2, 4, 2>(p, out, "qgemm_fast_256x256x128_w2x4_s2");
	case 34: return launch_fast<256, 128, 4, 2, 2>(p, out, "qgemm_fast_256x256x128_w4x2_s2");
	// 128 x 128 tiles for outputs too small to give every CU a 256 x 256 tile
	case 41:
		if (p.K % 128 != 0) return launch_fast<128, 128, 2, 2, 2, true>(p, out, "qgemm_fast_128x128x128_w2x2_s2_ktail");
		return launch_fast<128, 128, 2, 2, 2>(p, out, "qgemm_fast_128x128x128_w2x2_s2");
	case 42: return launch_fast<128, 128, 2, 2, 3>(p, out, "qgemm_fast_128x128x128_w2x2_s3");
	case 43: return launch_fast<128, 64, 2, 2, 3>(p, out, "qgemm_fast_128x128x64_w2x2_s3");
	case 44: return launch_fast<128, 64, 2, 2, 4>(p, out, "qgemm_fast_128x128x64_w2x2_s4");
	default: return -1;
	}
}

}  // namespace lten_hip
