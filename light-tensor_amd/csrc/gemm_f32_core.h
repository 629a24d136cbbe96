// The fp32 MFMA tile loop shared by the plain GEMM and the implicit-GEMM convolution kernels.
//
// One workgroup (WM x WN wavefronts) accumulates a BM x BN tile over `KT` steps of BK along the
// reduction dimension.  Operand values come from two callables, fetch_a(row, k, inside) and fetch_b(row, k, inside)
// (row inside the tile, k = global reduction index; they load from an address clamped into the operand whatever the
// position and set `inside` to whether the position exists: the core replaces the others by zeros), so that a
// kernel can hand in plain strided loads or im2col index arithmetic.  Tiles are staged through LDS in
// two buffers: the values of step kt+1 are fetched into registers before the MFMAs of step kt and
// written to the other buffer after them, one barrier per step.
//
// LDS layout follows the operand's layout in memory so that both the global fetch and the LDS store
// run along the thread index:
//   ROW_CONTIG (operand contiguous along its row index m or n): tile[k][ROWS + 4], threads walk rows
//   otherwise  (operand contiguous along k):                     tile[row][BK + 1],  threads walk k
#pragma once

#include <hip/hip_runtime.h>

namespace lten_hip {

typedef float v16f __attribute__((ext_vector_type(16)));

template <int ROWS, int BK, bool ROW_CONTIG>
struct TileLayout {
	static constexpr int LD = ROW_CONTIG ? ROWS + 4 : BK + 1;
	static constexpr int SIZE = ROW_CONTIG ? BK * LD : ROWS * LD;
	__device__ static __forceinline__ int at(int row, int k) { return ROW_CONTIG ? k * LD + row : row * LD + k; }
	// element e of the tile in thread order: the contiguous dimension moves fastest
	__device__ static __forceinline__ int row_of(int e) { return ROW_CONTIG ? e % ROWS : e / BK; }
	__device__ static __forceinline__ int k_of(int e) { return ROW_CONTIG ? e / ROWS : e % BK; }
};

template <int BM, int BN, int BK, int WM, int WN, bool A_ROW_CONTIG, bool B_ROW_CONTIG>
struct GemmCore {
	static constexpr int T = WM * WN * 64;
	static constexpr int TM = BM / WM, TN = BN / WN;
	static constexpr int FM = TM / 32, FN = TN / 32;
	typedef TileLayout<BM, BK, A_ROW_CONTIG> LA;
	typedef TileLayout<BN, BK, B_ROW_CONTIG> LB;
	static constexpr int A_PER_T = (BM * BK + T - 1) / T, B_PER_T = (BN * BK + T - 1) / T;
	static constexpr int LDS_FLOATS = 2 * (LA::SIZE + LB::SIZE);
	static_assert(TM % 32 == 0 && TN % 32 == 0 && BK % 2 == 0, "tile shape");

	// acc[i][j][4q + e] of lane (lrow = lane % 32, lk = lane / 32) of wave (wm, wn) is the tile element
	//   row = wm*TM + i*32 + 8q + 4*lk + e,  col = wn*TN + j*32 + lrow.
	template <typename FA, typename FB>
	__device__ static __forceinline__ void run(float* lds, int k_begin, int k_end, FA fetch_a, FB fetch_b, v16f (&acc)[FM][FN])
	{
		// The two buffers as offsets from the one LDS pointer: picked from an array of pointers they would lose their
		// address space, and the operand reads would become flat loads, which count as memory loads too and make
		// every MFMA wait for the prefetched step.
		constexpr int STAGE = LA::SIZE + LB::SIZE;
		const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
		const int wm = wave / WN, wn = wave % WN;
		const int lrow = lane & 31, lk = lane >> 5;
		float ra[A_PER_T], rb[B_PER_T];
		unsigned keep_a = 0, keep_b = 0;  // bit i: value i lies inside its operand
		static_assert(A_PER_T <= 32 && B_PER_T <= 32, "one bit per staged value");

		// Every load is issued, whatever the position (the callables clamp their addresses into the operand and say
		// through `inside` whether the position exists); what lies outside becomes zero on the way into LDS, a whole
		// MFMA loop later.  A load under a condition, or a select right behind it (which the compiler turns into one),
		// makes the compiler wait for every load in flight at once, the prefetched step included.
		auto load_global = [&](int k0) {
			keep_a = 0;
			keep_b = 0;
#pragma unroll
			for (int i = 0; i < A_PER_T; i++) {
				const int e = min(tid + i * T, BM * BK - 1);
				bool inside;
				ra[i] = fetch_a(LA::row_of(e), k0 + LA::k_of(e), inside);
				keep_a |= (unsigned)(inside & (tid + i * T < BM * BK)) << i;
			}
#pragma unroll
			for (int i = 0; i < B_PER_T; i++) {
				const int e = min(tid + i * T, BN * BK - 1);
				bool inside;
				rb[i] = fetch_b(LB::row_of(e), k0 + LB::k_of(e), inside);
				keep_b |= (unsigned)(inside & (tid + i * T < BN * BK)) << i;
			}
		};
		auto store_lds = [&](int buf) {
#pragma unroll
			for (int i = 0; i < A_PER_T; i++) {
				int e = tid + i * T;
				if (e < BM * BK) lds[buf * STAGE + LA::at(LA::row_of(e), LA::k_of(e))] = (keep_a >> i & 1) ? ra[i] : 0.0f;
			}
#pragma unroll
			for (int i = 0; i < B_PER_T; i++) {
				int e = tid + i * T;
				if (e < BN * BK) lds[buf * STAGE + LA::SIZE + LB::at(LB::row_of(e), LB::k_of(e))] = (keep_b >> i & 1) ? rb[i] : 0.0f;
			}
		};
		auto multiply = [&](int cur) {
#pragma unroll
			for (int kk = 0; kk < BK; kk += 2) {
				float fa[FM], fb[FN];
#pragma unroll
				for (int i = 0; i < FM; i++) fa[i] = lds[cur * STAGE + LA::at(wm * TM + i * 32 + lrow, kk + lk)];
#pragma unroll
				for (int j = 0; j < FN; j++) fb[j] = lds[cur * STAGE + LA::SIZE + LB::at(wn * TN + j * 32 + lrow, kk + lk)];
#pragma unroll
				for (int i = 0; i < FM; i++)
#pragma unroll
					for (int j = 0; j < FN; j++)
						acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
			}
		};

#pragma unroll
		for (int i = 0; i < FM; i++)
#pragma unroll
			for (int j = 0; j < FN; j++)
#pragma unroll
				for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

		if (k_begin >= k_end) return;
		load_global(k_begin);
		store_lds(0);
		__syncthreads();
		int cur = 0;
		// the last step is peeled: no fetch of the loop sits under a condition
		for (int k0 = k_begin; k0 + BK < k_end; k0 += BK) {
			load_global(k0 + BK);
			multiply(cur);
			store_lds(cur ^ 1);
			__syncthreads();
			cur ^= 1;
		}
		multiply(cur);
	}

	// Replaces every accumulator of this lane by f(row, col, value).
	template <typename F>
	__device__ static __forceinline__ void transform(v16f (&acc)[FM][FN], F f)
	{
		const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
		const int wm = wave / WN, wn = wave % WN;
		const int lrow = lane & 31, lk = lane >> 5;
#pragma unroll
		for (int j = 0; j < FN; j++)
#pragma unroll
			for (int i = 0; i < FM; i++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					acc[i][j][r] = f(wm * TM + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3), wn * TN + j * 32 + lrow, acc[i][j][r]);
	}

	// Visits every accumulator of this lane with its tile coordinates.
	template <typename F>
	__device__ static __forceinline__ void for_each(v16f (&acc)[FM][FN], F f)
	{
		const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
		const int wm = wave / WN, wn = wave % WN;
		const int lrow = lane & 31, lk = lane >> 5;
#pragma unroll
		for (int j = 0; j < FN; j++)
#pragma unroll
			for (int i = 0; i < FM; i++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					f(wm * TM + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3), wn * TN + j * 32 + lrow, acc[i][j][r]);
	}
};

}  // namespace lten_hip
