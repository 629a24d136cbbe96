// The fp32 MFMA tile loop shared by the plain GEMM and the implicit-GEMM convolution kernels.
//
// One workgroup (WM x WN wavefronts) accumulates a BM x BN tile over `KT` steps of BK along the
// reduction dimension.  Operand values come from two callables, fetch_a(row, k) and fetch_b(row, k)
// (row inside the tile, k = global reduction index; out-of-range positions must return 0), so that a
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
		float* sA[2] = { lds, lds + LA::SIZE + LB::SIZE };
		float* sB[2] = { lds + LA::SIZE, lds + 2 * LA::SIZE + LB::SIZE };
		const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
		const int wm = wave / WN, wn = wave % WN;
		const int lrow = lane & 31, lk = lane >> 5;
		float ra[A_PER_T], rb[B_PER_T];

		auto load_global = [&](int k0) {
#pragma unroll
			for (int i = 0; i < A_PER_T; i++) {
				int e = tid + i * T;
				ra[i] = (e < BM * BK) ? fetch_a(LA::row_of(e), k0 + LA::k_of(e)) : 0.0f;
			}
#pragma unroll
			for (int i = 0; i < B_PER_T; i++) {
				int e = tid + i * T;
				rb[i] = (e < BN * BK) ? fetch_b(LB::row_of(e), k0 + LB::k_of(e)) : 0.0f;
			}
		};
		auto store_lds = [&](int buf) {
#pragma unroll
			for (int i = 0; i < A_PER_T; i++) {
				int e = tid + i * T;
				if (e < BM * BK) sA[buf][LA::at(LA::row_of(e), LA::k_of(e))] = ra[i];
			}
#pragma unroll
			for (int i = 0; i < B_PER_T; i++) {
				int e = tid + i * T;
				if (e < BN * BK) sB[buf][LB::at(LB::row_of(e), LB::k_of(e))] = rb[i];
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
		for (int k0 = k_begin; k0 < k_end; k0 += BK) {
			const bool more = k0 + BK < k_end;
			if (more) load_global(k0 + BK);
#pragma unroll
			for (int kk = 0; kk < BK; kk += 2) {
				float fa[FM], fb[FN];
#pragma unroll
				for (int i = 0; i < FM; i++) fa[i] = sA[cur][LA::at(wm * TM + i * 32 + lrow, kk + lk)];
#pragma unroll
				for (int j = 0; j < FN; j++) fb[j] = sB[cur][LB::at(wn * TN + j * 32 + lrow, kk + lk)];
#pragma unroll
				for (int i = 0; i < FM; i++)
#pragma unroll
					for (int j = 0; j < FN; j++)
						acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
			}
			if (more) store_lds(cur ^ 1);
			__syncthreads();
			cur ^= 1;
		}
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
