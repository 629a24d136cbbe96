// fp32 GEMM for gfx950: the row-major sgemm that stands in for every cublasSgemm call of l-ten's GPU
// branches (l-ten/fully_connected.cpp:150,165; l-ten/md_array_cuda.h:513; l-ten/backprop.cpp:562,580,
// 2228,2252,2267) with the contract of cpu_gemm<float> (l-ten/math_fns.cpp:1258) plus leading dimensions.
//
// The tile loop lives in gemm_f32_core.h (32x32x2 fp32 MFMA blocks, LDS double buffer); this file adds
// the strided operand fetch, the alpha/beta/bias epilogue, the two degenerate shapes l-ten uses (K == 1
// rank-1 bias update, M == 1 column sum) and the dispatch.
#include "common.h"
#include "gemm_f32_core.h"
#include "sgemm_common.h"

#include <algorithm>

namespace lten_hip {


template <int BM, int BN, int BK, int WM, int WN, bool TA, bool TB>
__global__ __launch_bounds__(WM* WN * 64) void sgemm_kernel(SProblem p)
{
	// A[m][k] is at A[m*lda + k] (not transposed, contiguous in k) or A[k*lda + m] (transposed).
	// B[k][n] is at B[k*ldb + n] (not transposed, contiguous in n) or B[n*ldb + k] (transposed).
	typedef GemmCore<BM, BN, BK, WM, WN, TA, !TB> Core;
	__shared__ float lds[Core::LDS_FLOATS];

	const int tiles_n = (p.N + BN - 1) / BN;
	const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;
	const float* A = p.A + (int64_t)blockIdx.z * p.stride_a;
	const float* B = p.B + (int64_t)blockIdx.z * p.stride_b;
	float* C = p.C + (int64_t)blockIdx.z * p.stride_c;

	auto fetch_a = [&](int row, int k, bool& inside) -> float {
		inside = (m0 + row < p.M) & (k < p.K);
		const int m = min(m0 + row, p.M - 1), kc = min(k, p.K - 1);
		return TA ? A[(int64_t)kc * p.lda + m] : A[(int64_t)m * p.lda + kc];
	};
	auto fetch_b = [&](int row, int k, bool& inside) -> float {
		inside = (n0 + row < p.N) & (k < p.K);
		const int n = min(n0 + row, p.N - 1), kc = min(k, p.K - 1);
		return TB ? B[(int64_t)n * p.ldb + kc] : B[(int64_t)kc * p.ldb + n];
	};

	v16f acc[Core::FM][Core::FN];
	Core::run(lds, 0, p.K, fetch_a, fetch_b, acc);

	Core::for_each(acc, [&](int row, int col, float v) {
		const int m = m0 + row, n = n0 + col;
		if (m >= p.M || n >= p.N) return;
		float* c = C + (int64_t)m * p.ldc + n;
		float out = p.alpha * v;
		if (p.beta != 0.0f) out += p.beta * *c;  // beta == 0 overwrites: NaN/Inf in C must not survive
		if (p.bias) out += p.bias[n];
		sgemm_store(p, c, out);
	});
}

// Row sums of op(A) from the 32x32 kernels: every lane (row lrow, k-half g) of every wavefront has added the
// values it fed to the MFMAs; the 2 * WAVES shares of a row meet in LDS (scratch, at least 2 * WAVES * 32 floats
// that nothing else uses any more) and are added in a fixed order into rowsum[m0 + row].
template <int WAVES>
__device__ __forceinline__ void add_row_sums(float* scratch, float asum, float* rowsum, int m0, int M)
{
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	__syncthreads();
	scratch[(wave * 2 + (lane >> 5)) * 32 + (lane & 31)] = asum;
	__syncthreads();
	if (tid < 32 && m0 + tid < M) {
		float s = 0.0f;
#pragma unroll
		for (int i = 0; i < 2 * WAVES; i++) s += scratch[i * 32 + tid];
		rowsum[m0 + tid] += s;
	}
}

// Small outputs with a long K (the FullyConnected GEMMs at batch 128): one workgroup per 32x32 output tile,
// its WAVES wavefronts each reduce an interleaved share of K with operands loaded straight from global
// memory in the MFMA lane layout — no LDS staging, no barrier in the loop, loads unrolled ahead of their use —
// and the WAVES partial tiles meet in LDS, where they are added in wavefront order (deterministic).
// A k-contiguous operand is fetched 16 bytes per lane: lane (row, g) takes k = base + 4g .. 4g+3 and feeds the
// t-th of four MFMAs with element t; the other layout is fetched one dword per MFMA (two 128-byte rows per
// wave-wide load).  The assignment of k to MFMA slots is the same for A and B, which is all a dot product needs.
// `block`: index of the 32x32 output tile, `z`: batch index, `part`: WAVES * 1024 floats of LDS.
template <int WAVES, bool TA, bool TB>
__device__ __forceinline__ void sgemm_direct_body(const SProblem& p, int block, int z, float (*part)[32 * 32])
{
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int lrow = lane & 31, g = lane >> 5;
	const int tiles_n = (p.N + 31) / 32;
	const int m0 = (block / tiles_n) * 32, n0 = (block % tiles_n) * 32;
	const float* A = p.A + (int64_t)z * p.stride_a;
	const float* B = p.B + (int64_t)z * p.stride_b;
	float* C = p.C + (int64_t)z * p.stride_c;
	const int m = m0 + lrow, n = n0 + lrow;
	const bool mok = m < p.M, nok = n < p.N;
	const bool a_vec = !TA && (p.lda & 3) == 0 && (reinterpret_cast<uintptr_t>(A) & 15) == 0;
	const bool b_vec = TB && (p.ldb & 3) == 0 && (reinterpret_cast<uintptr_t>(B) & 15) == 0;

	v16f acc;
#pragma unroll
	for (int r = 0; r < 16; r++) acc[r] = 0.0f;
	float asum = 0.0f;  // this lane's share of row m of op(A)

	// groups of 8 consecutive k, dealt round-robin to the wavefronts
	const int groups = (p.K + 7) / 8;
#pragma unroll 4
	for (int grp = wave; grp < groups; grp += WAVES) {
		const int k = grp * 8 + g * 4;
		float a[4] = { 0.f, 0.f, 0.f, 0.f }, b[4] = { 0.f, 0.f, 0.f, 0.f };
		if (mok) {
			if (a_vec && k + 4 <= p.K) {
				const float4 v = *reinterpret_cast<const float4*>(A + (int64_t)m * p.lda + k);
				a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
			} else {
#pragma unroll
				for (int t = 0; t < 4; t++)
					if (k + t < p.K) a[t] = TA ? A[(int64_t)(k + t) * p.lda + m] : A[(int64_t)m * p.lda + k + t];
			}
		}
		if (nok) {
			if (b_vec && k + 4 <= p.K) {
				const float4 v = *reinterpret_cast<const float4*>(B + (int64_t)n * p.ldb + k);
				b[0] = v.x; b[1] = v.y; b[2] = v.z; b[3] = v.w;
			} else {
#pragma unroll
				for (int t = 0; t < 4; t++)
					if (k + t < p.K) b[t] = TB ? B[(int64_t)n * p.ldb + k + t] : B[(int64_t)(k + t) * p.ldb + n];
			}
		}
		asum += (a[0] + a[1]) + (a[2] + a[3]);
#pragma unroll
		for (int t = 0; t < 4; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc, 0, 0, 0);
	}

	// register 4q + e of lane (lrow, g): row 8q + 4g + e, column lrow
#pragma unroll
	for (int r = 0; r < 16; r++) part[wave][((r >> 2) * 8 + g * 4 + (r & 3)) * 32 + lrow] = acc[r];
	__syncthreads();
	for (int idx = tid; idx < 32 * 32; idx += WAVES * 64) {
		const int row = idx >> 5, col = idx & 31;
		if (m0 + row >= p.M || n0 + col >= p.N) continue;
		float sum = 0.0f;
#pragma unroll
		for (int w = 0; w < WAVES; w++) sum += part[w][idx];
		float* c = C + (int64_t)(m0 + row) * p.ldc + n0 + col;
		float out = p.alpha * sum;
		if (p.beta != 0.0f) out += p.beta * *c;
		if (p.bias) out += p.bias[n0 + col];
		sgemm_store(p, c, out);
	}
	if (p.rowsum != nullptr && n0 == 0) add_row_sums<WAVES>(&part[0][0], asum, p.rowsum, m0, p.M);
}

template <int WAVES, bool TA, bool TB>
__global__ __launch_bounds__(WAVES * 64) void sgemm_direct_kernel(SProblem p)
{
	__shared__ float part[WAVES][32 * 32];
	sgemm_direct_body<WAVES, TA, TB>(p, blockIdx.x, blockIdx.z, part);
}

// The same decomposition with whole cache lines per load: the direct kernel above asks the texture addresser for 32
// different lines per wave-wide load (32 rows x 32 bytes), which is what bounds it at these sizes.  Here a wave-wide
// 16-byte load covers 8 rows x 128 bytes along the operand's contiguous dimension (8 lines), the values pass through
// a wavefront-private LDS slab (no barrier: LDS operations of one wavefront complete in order) and come back in
// the MFMA lane layout.  A batch is 32 k-values; wavefront w takes batches w, w + WAVES, ...; the loads of up to
// UB batches are in flight at once.  Operand rows of 36 floats keep both the 16-byte stores and the reads free of
// bank conflicts.  Used when the operands allow 16-byte loads (leading dimensions and bases multiples of 4 floats).
template <int WAVES>
struct StagedLds {
	static constexpr int LD = 36, SLAB = 32 * LD;
	static constexpr int FLOATS = WAVES * 2 * SLAB > WAVES * 1024 ? WAVES * 2 * SLAB : WAVES * 1024;
};

// `block`: index of the 32x32 output tile, `z`: batch index, `lds`: StagedLds<WAVES>::FLOATS floats, 16-byte aligned.
template <int WAVES, bool TA, bool TB>
__device__ __forceinline__ void sgemm_staged_body(const SProblem& p, int block, int z, float* lds)
{
	constexpr int UB = 4, LD = StagedLds<WAVES>::LD, SLAB = StagedLds<WAVES>::SLAB;
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int lrow = lane & 31, g = lane >> 5;
	const int tiles_n = (p.N + 31) / 32;
	const int m0 = (block / tiles_n) * 32, n0 = (block % tiles_n) * 32;
	const float* A = p.A + (int64_t)z * p.stride_a;
	const float* B = p.B + (int64_t)z * p.stride_b;
	float* C = p.C + (int64_t)z * p.stride_c;
	float* sA = lds + wave * 2 * SLAB;
	float* sB = sA + SLAB;
	const int r8 = lane >> 3, c4 = (lane & 7) * 4;  // this lane's row within a group of 8 and its 4-float column

	v16f acc;
#pragma unroll
	for (int r = 0; r < 16; r++) acc[r] = 0.0f;
	float asum = 0.0f;  // this lane's share of row m0 + lrow of op(A)

	// one operand, one batch: four 16-byte loads per lane
	auto fetch = [&](const float* base, int64_t ld, bool k_contig, int rows_limit, int row0, int k0, float4 (&v)[4]) {
#pragma unroll
		for (int i = 0; i < 4; i++) {
			const int q = 8 * i + r8;  // k_contig: tile row, else: k offset inside the batch
			v[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (k_contig) {
				const int row = row0 + q, k = k0 + c4;
				if (row < rows_limit && k < p.K) {
					const float* src = base + (int64_t)row * ld + k;
					if (k + 3 < p.K) v[i] = *reinterpret_cast<const float4*>(src);
					else { v[i].x = src[0]; if (k + 1 < p.K) v[i].y = src[1]; if (k + 2 < p.K) v[i].z = src[2]; }
				}
			} else {
				const int k = k0 + q, col = row0 + c4;
				if (k < p.K && col < rows_limit) {
					const float* src = base + (int64_t)k * ld + col;
					if (col + 3 < rows_limit) v[i] = *reinterpret_cast<const float4*>(src);
					else { v[i].x = src[0]; if (col + 1 < rows_limit) v[i].y = src[1]; if (col + 2 < rows_limit) v[i].z = src[2]; }
				}
			}
		}
	};
	// slab layouts: k-contiguous operand [tile row][k], the other [k][tile row]; both rows of LD floats
	auto stage = [&](float* slab, const float4 (&v)[4]) {
#pragma unroll
		for (int i = 0; i < 4; i++) *reinterpret_cast<float4*>(slab + (8 * i + r8) * LD + c4) = v[i];
	};

	const int batches = (p.K + 31) / 32;
	for (int b0 = wave; b0 < batches; b0 += WAVES * UB) {
		float4 va[UB][4], vb[UB][4];
#pragma unroll
		for (int u = 0; u < UB; u++) {
			const int b = b0 + u * WAVES;
			if (b < batches) {
				fetch(A, p.lda, !TA, p.M, m0, b * 32, va[u]);
				fetch(B, p.ldb, TB, p.N, n0, b * 32, vb[u]);
			}
		}
#pragma unroll
		for (int u = 0; u < UB; u++) {
			if (b0 + u * WAVES >= batches) break;
			stage(sA, va[u]);
			stage(sB, vb[u]);
#pragma unroll
			for (int q = 0; q < 4; q++) {
				// MFMA step (q, t) multiplies k = 8q + 4g + t of the batch
				float a[4], bb[4];
				if (!TA) {
					const float4 t4 = *reinterpret_cast<const float4*>(sA + lrow * LD + 8 * q + 4 * g);
					a[0] = t4.x; a[1] = t4.y; a[2] = t4.z; a[3] = t4.w;
				} else {
#pragma unroll
					for (int t = 0; t < 4; t++) a[t] = sA[(8 * q + 4 * g + t) * LD + lrow];
				}
				if (TB) {
					const float4 t4 = *reinterpret_cast<const float4*>(sB + lrow * LD + 8 * q + 4 * g);
					bb[0] = t4.x; bb[1] = t4.y; bb[2] = t4.z; bb[3] = t4.w;
				} else {
#pragma unroll
					for (int t = 0; t < 4; t++) bb[t] = sB[(8 * q + 4 * g + t) * LD + lrow];
				}
				asum += (a[0] + a[1]) + (a[2] + a[3]);
#pragma unroll
				for (int t = 0; t < 4; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], bb[t], acc, 0, 0, 0);
			}
		}
	}

	// the wavefronts' partial tiles meet in LDS (the slabs are no longer needed) and are added in wavefront order
	__syncthreads();
#pragma unroll
	for (int r = 0; r < 16; r++) lds[wave * 1024 + ((r >> 2) * 8 + g * 4 + (r & 3)) * 32 + lrow] = acc[r];
	__syncthreads();
	for (int idx = tid; idx < 32 * 32; idx += WAVES * 64) {
		const int row = idx >> 5, col = idx & 31;
		if (m0 + row >= p.M || n0 + col >= p.N) continue;
		float sum = 0.0f;
#pragma unroll
		for (int w = 0; w < WAVES; w++) sum += lds[w * 1024 + idx];
		float* c = C + (int64_t)(m0 + row) * p.ldc + n0 + col;
		float out = p.alpha * sum;
		if (p.beta != 0.0f) out += p.beta * *c;
		if (p.bias) out += p.bias[n0 + col];
		sgemm_store(p, c, out);
	}
	if (p.rowsum != nullptr && n0 == 0) add_row_sums<WAVES>(lds, asum, p.rowsum, m0, p.M);
}

template <int WAVES, bool TA, bool TB>
__global__ __launch_bounds__(WAVES * 64) void sgemm_staged_kernel(SProblem p)
{
	__shared__ __attribute__((aligned(16))) float lds[StagedLds<WAVES>::FLOATS];
	sgemm_staged_body<WAVES, TA, TB>(p, blockIdx.x, blockIdx.z, lds);
}

// Both products of FullyConnected backward in one launch: the first `blocks_x` workgroups compute tiles of
// dX = dY W (NN), the others tiles of dW = dY^T X (TN, with the bias gradient as its row sums), both with the
// direct body (32 KB of LDS, four workgroups per CU).  The two are independent and each fills the chip for a few
// microseconds only, so a launch of their own for each costs about as much again as the work.  The whole-line
// body is not used here: its 74 KB of LDS would halve the number of resident workgroups for both products
// (measured at batch 128, 1024 -> 1024: 18.6 us with it, 14.8 without, 17.9 as two launches).
__global__ __launch_bounds__(512) void sgemm_fc_backward_pair_kernel(SProblem px, SProblem pw, int blocks_x)
{
	__shared__ float part[8][32 * 32];
	if ((int)blockIdx.x < blocks_x) sgemm_direct_body<8, false, false>(px, blockIdx.x, 0, part);
	else sgemm_direct_body<8, true, false>(pw, blockIdx.x - blocks_x, 0, part);
}

// The pair above for the last layer of a classifier, with the loss in front: every workgroup works out the gradient
// of the loss with respect to the logits (log_softmax, nll_loss and their backward functions: a few thousand values)
// into LDS for itself and reads the dY operand of its tile from there, so the loss needs no launch of its own and no
// hand-over between workgroups; one workgroup also writes the log-probabilities, that gradient and the loss.
// Sixteen lanes per row, one per column: max and sums over the row in the order of the separate kernels (pairs 8
// apart, then 4, 2, 1, lanes past the row holding zeros), the loss summed as nll_loss_kernel sums it (1024 strided
// shares, here two per thread; wavefront trees; 16 partial sums in order): every value is bit-identical to what
// lten_hip_log_softmax_nll_loss_grad_f32 followed by lten_hip_fc_backward_f32 gives.
struct LossRows {
	int rows, cols;  // rows * cols <= 4096, cols <= 16
	const float* x;  // logits [rows][cols]
	const float* target;
	float alpha, loss_scale;
	float* y;  // log-probabilities
	float* loss;
	float* dx;  // gradient with respect to the logits
};

// Sum and maximum over the 16 lanes of a row by rotations within the row in the vector ALU (DPP row_ror:8, 4, 2, 1).
// Every lane ends with the same value: pairs 8 apart, then pairs of pairs 4 apart, 2, 1 — the tree the separate kernels
// build with lane exchanges, operands commuted at most.
template <int CTRL>
__device__ __forceinline__ float row_rotate(float v)
{
	return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

__device__ __forceinline__ float row16_sum(float v)
{
	v += row_rotate<0x128>(v);
	v += row_rotate<0x124>(v);
	v += row_rotate<0x122>(v);
	v += row_rotate<0x121>(v);
	return v;
}

__device__ __forceinline__ float row16_max(float v)
{
	v = fmaxf(v, row_rotate<0x128>(v));
	v = fmaxf(v, row_rotate<0x124>(v));
	v = fmaxf(v, row_rotate<0x122>(v));
	v = fmaxf(v, row_rotate<0x121>(v));
	return v;
}

__global__ __launch_bounds__(512) void sgemm_fc_backward_pair_loss_kernel(SProblem px, SProblem pw, int blocks_x, LossRows L)
{
	__shared__ float part[8][32 * 32];
	__shared__ float sdy[4096];
	__shared__ float part16[16];
	const int tid = threadIdx.x, c = tid & 15;
	// A tile of dX needs the 32 rows of its own row block; a tile of dW needs them all, and the first of those writes
	// the loss outputs as well.
	const bool for_x = (int)blockIdx.x < blocks_x;
	const bool first = (int)blockIdx.x == blocks_x;
	float* logp = &part[0][0];  // free until the tile's partial sums are exchanged
	auto rows_from = [&](int r) {
		const bool ok = r < L.rows && c < L.cols;
		const float xv = ok ? L.x[r * L.cols + c] : -INFINITY;
		const float tv = ok ? L.target[r * L.cols + c] : 0.0f;
		const float m = row16_max(xv);
		const float e = ok ? expf(xv - m) : 0.0f;
		const float s = row16_sum(e);
		const float lp = logf(e / s);
		const float dy = ok ? L.alpha * tv : 0.0f;
		const float sd = row16_sum(dy);
		const float g = dy - expf(lp) * sd;
		if (ok) {
			sdy[r * L.cols + c] = g;
			if (first) {
				L.y[r * L.cols + c] = lp;
				L.dx[r * L.cols + c] = g;
				logp[r * L.cols + c] = lp;
			}
		}
	};
	if (for_x) {
		const int tiles_n = (px.N + 31) / 32;
		rows_from(((int)blockIdx.x / tiles_n) * 32 + (tid >> 4));
	} else {
		// four rows per thread at a time: independent chains of exchanges and transcendentals that overlap
		for (int r0 = 0; r0 < L.rows; r0 += 128) {
#pragma unroll
			for (int u = 0; u < 4; u++) rows_from(r0 + 32 * u + (tid >> 4));
		}
	}
	__syncthreads();
	if (first) {
		const int len = L.rows * L.cols;
#pragma unroll
		for (int v = 0; v < 2; v++) {
			const int vt = tid + 512 * v;
			float acc = 0.0f;
			for (int i = vt; i < len; i += 1024) acc += logp[i] * L.target[i];
#pragma unroll
			for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
			if ((tid & 63) == 0) part16[vt >> 6] = acc;
		}
		__syncthreads();
		if (tid == 0) {
			float tot = 0.0f;
#pragma unroll
			for (int w = 0; w < 16; w++) tot += part16[w];
			*L.loss = tot * L.loss_scale;
		}
	}
	SProblem qx = px, qw = pw;
	qx.A = sdy;
	qw.A = sdy;
	if ((int)blockIdx.x < blocks_x) sgemm_direct_body<8, false, false>(qx, blockIdx.x, 0, part);
	else sgemm_direct_body<8, true, false>(qw, blockIdx.x - blocks_x, 0, part);
}

// C = A^T B (TN) with a short K (the weight gradient dW = dY^T X at a small batch): a 32x32 output tile per wavefront
// over the whole K, operands straight from global memory in the MFMA lane layout (both are read along their contiguous
// dimension: two 128-byte rows per wave-wide load), the loads of eight groups of 8 k in flight together, no LDS, no
// barrier — cutting a K of 128 over eight wavefronts leaves each with two groups and a workgroup with more exchange than
// arithmetic.  `tile` counts 32x32 tiles row-major.  The wavefronts of the first column tile add the row sums of op(A)
// into p.rowsum.
__device__ __forceinline__ void sgemm_tn_wave_tile(const SProblem& p, int tile)
{
	const int lane = threadIdx.x & 63, lrow = lane & 31, g = lane >> 5;
	const int tiles_n = (p.N + 31) / 32;
	const int m0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
	if (m0 >= p.M) return;
	const int m = m0 + lrow, n = n0 + lrow;
	const bool mok = m < p.M, nok = n < p.N;
	const float* a_col = p.A + (mok ? m : 0);
	const float* b_col = p.B + (nok ? n : 0);
	v16f acc;
#pragma unroll
	for (int r = 0; r < 16; r++) acc[r] = 0.0f;
	float asum = 0.0f;
	const int groups = (p.K + 7) / 8;
	constexpr int U = 8;
	for (int g0 = 0; g0 < groups; g0 += U) {
		float a[U][4], b[U][4];
#pragma unroll
		for (int u = 0; u < U; u++) {
			const int k = (g0 + u) * 8 + g * 4;
#pragma unroll
			for (int t = 0; t < 4; t++) {
				// rows past K are not read; columns past M or N read column 0 and are never stored
				const int kk = k + t < p.K ? k + t : 0;
				const float av = a_col[(int64_t)kk * p.lda], bv = b_col[(int64_t)kk * p.ldb];
				a[u][t] = (k + t < p.K && mok) ? av : 0.0f;
				b[u][t] = (k + t < p.K && nok) ? bv : 0.0f;
			}
		}
#pragma unroll
		for (int u = 0; u < U; u++) {
			if (g0 + u >= groups) break;
			asum += (a[u][0] + a[u][1]) + (a[u][2] + a[u][3]);
#pragma unroll
			for (int t = 0; t < 4; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t], b[u][t], acc, 0, 0, 0);
		}
	}
	// register 4q + e of lane (lrow, g): row 8q + 4g + e, column lrow
	if (nok) {
#pragma unroll
		for (int r = 0; r < 16; r++) {
			const int row = m0 + (r >> 2) * 8 + g * 4 + (r & 3);
			if (row >= p.M) continue;
			float* c = p.C + (int64_t)row * p.ldc + n;
			float out = p.alpha * acc[r];
			if (p.beta != 0.0f) out += p.beta * *c;
			sgemm_store(p, c, out);
		}
	}
	if (p.rowsum != nullptr && n0 == 0) {
		const float s = asum + __shfl_xor(asum, 32, 64);
		if (g == 0 && mok) p.rowsum[m] += s;
	}
}

// The same tile with whole cache lines per load: a wave-wide 16-byte load covers 8 k-rows x 128 bytes of an operand (the
// loads above fetch 4 bytes per lane, two rows of 128 bytes per instruction: eight times as many instructions for the
// memory pipeline), the values pass through a wavefront-private LDS slab ([32 k][36] floats per operand; no barrier: LDS
// operations of one wavefront complete in order) and come back one float per MFMA in its lane layout.  The next batch
// of 32 k is in flight while the current one is multiplied.  Needs M % 4 == 0, N % 4 == 0, lda % 4 == 0, ldb % 4 == 0
// and 16-byte aligned operands.  `slab`: 2 * 32 * 36 floats of this wavefront.
__device__ __forceinline__ void sgemm_tn_wave_tile_lines(const SProblem& p, int tile, float* slab)
{
	constexpr int LD = 36;
	const int lane = threadIdx.x & 63, lrow = lane & 31, g = lane >> 5;
	const int kr = lane >> 3, c4 = (lane & 7) * 4;
	const int tiles_n = (p.N + 31) / 32;
	const int m0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
	if (m0 >= p.M) return;
	const bool a_ok = m0 + c4 < p.M, b_ok = n0 + c4 < p.N;
	const float* a_src = p.A + m0 + c4;
	const float* b_src = p.B + n0 + c4;
	float* sA = slab;
	float* sB = slab + 32 * LD;
	struct Batch {
		float4 a[4], b[4];
	};
	auto fetch = [&](int kb, Batch& v) {
#pragma unroll
		for (int i = 0; i < 4; i++) {
			const int k = kb + 8 * i + kr;
			v.a[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			v.b[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (k < p.K) {
				if (a_ok) v.a[i] = *reinterpret_cast<const float4*>(a_src + (int64_t)k * p.lda);
				if (b_ok) v.b[i] = *reinterpret_cast<const float4*>(b_src + (int64_t)k * p.ldb);
			}
		}
	};
	v16f acc;
#pragma unroll
	for (int r = 0; r < 16; r++) acc[r] = 0.0f;
	float asum = 0.0f;
	Batch cur, nxt;
	fetch(0, cur);
	for (int kb = 0; kb < p.K; kb += 32) {
		fetch(kb + 32, nxt);  // rows past K read as zeros without a load
#pragma unroll
		for (int i = 0; i < 4; i++) {
			*reinterpret_cast<float4*>(sA + (8 * i + kr) * LD + c4) = cur.a[i];
			*reinterpret_cast<float4*>(sB + (8 * i + kr) * LD + c4) = cur.b[i];
		}
#pragma unroll
		for (int s = 0; s < 16; s++) {
			const float fa = sA[(2 * s + g) * LD + lrow], fb = sB[(2 * s + g) * LD + lrow];
			asum += fa;
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc, 0, 0, 0);
		}
		cur = nxt;
	}
	const int m = m0 + lrow, n = n0 + lrow;
	// register 4q + e of lane (lrow, g): row 8q + 4g + e, column lrow
	if (n < p.N) {
#pragma unroll
		for (int r = 0; r < 16; r++) {
			const int row = m0 + (r >> 2) * 8 + g * 4 + (r & 3);
			if (row >= p.M) continue;
			float* c = p.C + (int64_t)row * p.ldc + n;
			float out = p.alpha * acc[r];
			if (p.beta != 0.0f) out += p.beta * *c;
			sgemm_store(p, c, out);
		}
	}
	if (p.rowsum != nullptr && n0 == 0) {
		const float sum = asum + __shfl_xor(asum, 32, 64);
		if (g == 0 && m < p.M) p.rowsum[m] += sum;
	}
}

// The same pair with the weight gradient on whole-K tiles per wavefront: eight of its tiles per workgroup.  LINES: the
// weight gradient's operands allow whole-line loads.
template <bool LINES>
__global__ __launch_bounds__(512) void sgemm_fc_backward_pair_shortk_kernel(SProblem px, SProblem pw, int blocks_x)
{
	constexpr int SLAB = 2 * 32 * 36;
	__shared__ __attribute__((aligned(16))) float lds[LINES ? 8 * SLAB : 8 * 32 * 32];
	const int wave = (int)(threadIdx.x >> 6);
	if ((int)blockIdx.x < blocks_x) sgemm_direct_body<8, false, false>(px, blockIdx.x, 0, reinterpret_cast<float (*)[32 * 32]>(lds));
	else if (LINES) sgemm_tn_wave_tile_lines(pw, ((int)blockIdx.x - blocks_x) * 8 + wave, lds + wave * SLAB);
	else sgemm_tn_wave_tile(pw, ((int)blockIdx.x - blocks_x) * 8 + wave);
}

// FullyConnected forward at small batch sizes: C[M x N] = A[M x K] B[N x K]^T with M <= 32, a stream over the
// weights B.  The 32x32 kernels above give such a product N / 32 workgroups; here a workgroup takes 16 columns
// (N / 16 workgroups: 256 for a 4096-wide layer) on 16x16x4 MFMA tiles, MB = 1 or 2 blocks of 16 activation rows.
// K is cut into batches of 32, dealt round-robin to the 8 wavefronts; a wave-wide 16-byte load covers 8 rows x 128
// bytes (whole cache lines), the values pass through a wavefront-private LDS slab (no barrier: LDS operations of one
// wavefront complete in order) and come back in the MFMA lane layout: lane (r = lane % 16, q = lane / 16) feeds row
// (or column) r with k = 16h + 4q + t for the MFMA number (h, t) of the batch, the same for both operands.  The loads
// of the next UB batches are in flight while the current UB are multiplied.
typedef float v4f __attribute__((ext_vector_type(4)));

// BT: B is [N x K] (the NT product above); otherwise B is [K x N], rows contiguous in n (the NN product, the data
// gradient dX = dY W of a FullyConnected layer): a wave-wide 16-byte load then covers 16 k-rows x 64 bytes of the
// column block, the slab holds [32 k][16 n] and the operand is read one float per MFMA (lane (n, q): k = 16h + 4q + t).
template <int MB, bool BT>
struct SkinnyShape {
	static constexpr int WAVES = 8, LD = 36, LDB = 20;
	static constexpr int A_SLAB = MB * 16 * LD, B_SLAB = BT ? 16 * LD : 32 * LDB;
	static constexpr int SLABS = WAVES * (A_SLAB + B_SLAB), TILES = WAVES * MB * 256;
	static constexpr int LDS_FLOATS = SLABS > TILES ? SLABS : TILES;
};

// col_block: which 16 columns, row_block: which MB * 16 rows; lds: SkinnyShape<MB, BT>::LDS_FLOATS floats
template <int MB, bool BT>
__device__ __forceinline__ void sgemm_skinny_body(const SProblem& p, int col_block, int row_block, float* lds)
{
	typedef SkinnyShape<MB, BT> S;
	constexpr int WAVES = S::WAVES, UB = 2, LD = S::LD, LDB = S::LDB;
	constexpr int A_SLAB = S::A_SLAB, B_SLAB = S::B_SLAB;
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int r16 = lane & 15, q4 = lane >> 4;
	const int r8 = lane >> 3, c4 = (lane & 7) * 4;
	const int k16 = lane >> 2, n4 = (lane & 3) * 4;  // NN: this lane's k-row within 16 and its four columns
	const int n0 = col_block * 16;
	const int mrow0 = row_block * (MB * 16);
	float* sA = lds + wave * (A_SLAB + B_SLAB);
	float* sB = sA + A_SLAB;

	v4f acc[MB];
#pragma unroll
	for (int b = 0; b < MB; b++) acc[b] = v4f{ 0.0f, 0.0f, 0.0f, 0.0f };

	struct Batch {
		float4 a[2 * MB], b[2];
	};
	// K % 4 == 0: a float4 lies inside K or outside as a whole.  Every load is issued, from an address clamped into the
	// operand, and what lies outside is replaced by zeros when the batch is multiplied: with the loads under conditions
	// the compiler can no longer count how many are in flight and waits for all of them before the first multiply, the
	// prefetched ones included.
	auto fetch = [&](int batch, Batch& v) {
		const int kc = min(batch * 32 + c4, p.K - 4);
#pragma unroll
		for (int i = 0; i < 2 * MB; i++)
			v.a[i] = *reinterpret_cast<const float4*>(p.A + (int64_t)min(mrow0 + 8 * i + r8, p.M - 1) * p.lda + kc);
#pragma unroll
		for (int i = 0; i < 2; i++) {
			if (BT) v.b[i] = *reinterpret_cast<const float4*>(p.B + (int64_t)min(n0 + 8 * i + r8, p.N - 1) * p.ldb + kc);
			else  // N % 4 == 0: the four columns are inside N or outside together
				v.b[i] = *reinterpret_cast<const float4*>(p.B + (int64_t)min(batch * 32 + 16 * i + k16, p.K - 1) * p.ldb + min(n0 + n4, p.N - 4));
		}
	};
	auto keep = [](const float4& t, bool in) { return make_float4(in ? t.x : 0.0f, in ? t.y : 0.0f, in ? t.z : 0.0f, in ? t.w : 0.0f); };
	auto multiply = [&](int batch, const Batch& v) {
		const bool k_in = batch * 32 + c4 < p.K;
#pragma unroll
		for (int i = 0; i < 2 * MB; i++) *reinterpret_cast<float4*>(sA + (8 * i + r8) * LD + c4) = keep(v.a[i], mrow0 + 8 * i + r8 < p.M && k_in);
#pragma unroll
		for (int i = 0; i < 2; i++) {
			if (BT) *reinterpret_cast<float4*>(sB + (8 * i + r8) * LD + c4) = keep(v.b[i], n0 + 8 * i + r8 < p.N && k_in);
			else *reinterpret_cast<float4*>(sB + (16 * i + k16) * LDB + n4) = keep(v.b[i], batch * 32 + 16 * i + k16 < p.K && n0 + n4 < p.N);
		}
#pragma unroll
		for (int h = 0; h < 2; h++) {
			float4 fb;
			if (BT) fb = *reinterpret_cast<const float4*>(sB + r16 * LD + 16 * h + 4 * q4);
			else {
				const float* col = sB + (16 * h + 4 * q4) * LDB + r16;
				fb = make_float4(col[0], col[LDB], col[2 * LDB], col[3 * LDB]);
			}
			// the row blocks take turns, so that consecutive MFMAs do not wait for each other's sums
			float4 fa[MB];
#pragma unroll
			for (int b = 0; b < MB; b++) fa[b] = *reinterpret_cast<const float4*>(sA + (16 * b + r16) * LD + 16 * h + 4 * q4);
#pragma unroll
			for (int b = 0; b < MB; b++) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[b].x, fb.x, acc[b], 0, 0, 0);
#pragma unroll
			for (int b = 0; b < MB; b++) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[b].y, fb.y, acc[b], 0, 0, 0);
#pragma unroll
			for (int b = 0; b < MB; b++) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[b].z, fb.z, acc[b], 0, 0, 0);
#pragma unroll
			for (int b = 0; b < MB; b++) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[b].w, fb.w, acc[b], 0, 0, 0);
		}
	};

	// No load stands under a condition (a load in a conditional block costs a wait for everything in flight at the first
	// use behind it): while a further round exists its batches are fetched, one past the end as the last one again, and
	// the round in hand is multiplied whole; the last round is multiplied as far as it exists, with no fetch beside it.
	const int batches = (p.K + 31) / 32;
	Batch cur[UB], nxt[UB];
	int b0 = wave;
#pragma unroll
	for (int u = 0; u < UB; u++) fetch(min(b0 + u * WAVES, batches - 1), cur[u]);
	for (; b0 + WAVES * UB < batches; b0 += WAVES * UB) {
#pragma unroll
		for (int u = 0; u < UB; u++) fetch(min(b0 + (UB + u) * WAVES, batches - 1), nxt[u]);
#pragma unroll
		for (int u = 0; u < UB; u++) multiply(b0 + u * WAVES, cur[u]);
#pragma unroll
		for (int u = 0; u < UB; u++) cur[u] = nxt[u];
	}
#pragma unroll
	for (int u = 0; u < UB; u++)
		if (b0 + u * WAVES < batches) multiply(b0 + u * WAVES, cur[u]);

	// accumulator register e of lane (r16, q4) of block b: row 16b + 4 q4 + e, column r16.  The wavefronts' partial
	// tiles meet in LDS (the slabs are no longer needed) and are added in wavefront order.
	__syncthreads();
#pragma unroll
	for (int b = 0; b < MB; b++)
#pragma unroll
		for (int e = 0; e < 4; e++) lds[wave * (MB * 256) + (16 * b + 4 * q4 + e) * 16 + r16] = acc[b][e];
	__syncthreads();
	for (int idx = tid; idx < MB * 256; idx += WAVES * 64) {
		const int row = mrow0 + (idx >> 4), col = idx & 15;
		if (row >= p.M || n0 + col >= p.N) continue;
		float sum = 0.0f;
#pragma unroll
		for (int w = 0; w < WAVES; w++) sum += lds[w * (MB * 256) + idx];
		float* c = p.C + (int64_t)row * p.ldc + n0 + col;
		float out = p.alpha * sum;
		if (p.beta != 0.0f) out += p.beta * *c;
		if (p.bias) out += p.bias[n0 + col];
		sgemm_store(p, c, out);
	}
}

template <int MB>
__global__ __launch_bounds__(512) void sgemm_skinny_nt_kernel(SProblem p)
{
	__shared__ __attribute__((aligned(16))) float lds[SkinnyShape<MB, true>::LDS_FLOATS];
	// (grid plane z: problem z of a strided batch)
	p.A += (int64_t)blockIdx.z * p.stride_a;
	p.B += (int64_t)blockIdx.z * p.stride_b;
	p.C += (int64_t)blockIdx.z * p.stride_c;
	sgemm_skinny_body<MB, true>(p, blockIdx.x, blockIdx.y, lds);
}

template <int MB>
__global__ __launch_bounds__(512) void sgemm_skinny_nn_kernel(SProblem p)
{
	__shared__ __attribute__((aligned(16))) float lds[SkinnyShape<MB, false>::LDS_FLOATS];
	// XCD x (consecutive workgroups go round-robin to the eight of them) takes a contiguous run of column blocks: a block
	// reads 64-byte pieces of B's rows, and neighbours that share those cache lines should share an L2 as well
	const int nblk = gridDim.x, bx = blockIdx.x & 7;
	const int blk = bx * (nblk >> 3) + min(bx, nblk & 7) + ((int)blockIdx.x >> 3);
	sgemm_skinny_body<MB, false>(p, blk, blockIdx.y, lds);
}

// sgemm_tn_wave_tile_lines over k in [k_begin, k_end) only, the sums left in `acc` and `asum` (this lane's share of the
// row sums of op(A)).
__device__ __forceinline__ void sgemm_tn_tile_lines_partial(const SProblem& p, int tile, int k_begin, int k_end, float* slab, v16f& acc, float& asum)
{
	constexpr int LD = 36;
	const int lane = threadIdx.x & 63, lrow = lane & 31, g = lane >> 5;
	const int kr = lane >> 3, c4 = (lane & 7) * 4;
	const int tiles_n = (p.N + 31) / 32;
	const int m0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
	const bool a_ok = m0 + c4 < p.M, b_ok = n0 + c4 < p.N;
	const float* a_src = p.A + m0 + c4;
	const float* b_src = p.B + n0 + c4;
	float* sA = slab;
	float* sB = slab + 32 * LD;
	struct Batch {
		float4 a[4], b[4];
	};
	auto fetch = [&](int kb, Batch& v) {
#pragma unroll
		for (int i = 0; i < 4; i++) {
			const int k = kb + 8 * i + kr;
			v.a[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			v.b[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (k < k_end) {
				if (a_ok) v.a[i] = *reinterpret_cast<const float4*>(a_src + (int64_t)k * p.lda);
				if (b_ok) v.b[i] = *reinterpret_cast<const float4*>(b_src + (int64_t)k * p.ldb);
			}
		}
	};
	Batch cur, nxt;
	fetch(k_begin, cur);
	for (int kb = k_begin; kb < k_end; kb += 32) {
		fetch(kb + 32, nxt);  // rows past the range read as zeros without a load
#pragma unroll
		for (int i = 0; i < 4; i++) {
			*reinterpret_cast<float4*>(sA + (8 * i + kr) * LD + c4) = cur.a[i];
			*reinterpret_cast<float4*>(sB + (8 * i + kr) * LD + c4) = cur.b[i];
		}
#pragma unroll
		for (int s = 0; s < 16; s++) {
			const float fa = sA[(2 * s + g) * LD + lrow], fb = sB[(2 * s + g) * LD + lrow];
			asum += fa;
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc, 0, 0, 0);
		}
		cur = nxt;
	}
}

// Both products of FullyConnected backward in one launch, each on as many workgroups as the chip has CUs: dW on the
// whole-line tiles, four per workgroup (wavefront w multiplies tile w % 4 over half w / 4 of the batch; the halves are
// added through LDS, the lower half first), dX on the weight-streaming tiles.  With 128 workgroups per product (eight
// whole-K tiles of dW, or one 32 x 32 tile of dX, per workgroup) each product kept half of the CUs busy for 11-13 us.
__global__ __launch_bounds__(512) void sgemm_fc_backward_pair_wide_kernel(SProblem px, SProblem pw, int blocks_w, int tiles_w, int cols_x)
{
	constexpr int SLAB = 2 * 32 * 36;
	constexpr int FLOATS = SkinnyShape<2, false>::LDS_FLOATS > 8 * SLAB ? SkinnyShape<2, false>::LDS_FLOATS : 8 * SLAB;
	static_assert(8 * SLAB >= 4 * 16 * 64 + 4 * 32, "the exchange of the halves fits the slabs");
	__shared__ __attribute__((aligned(16))) float lds[FLOATS];
	if ((int)blockIdx.x >= blocks_w) {
		// Consecutive workgroups go round-robin to the eight XCDs, each with an L2 of its own.  XCD x takes a contiguous
		// run of the (column block, row block) pairs in column-major order, i.e. a range of column blocks with all their
		// row blocks: a column block reads 64-byte pieces of the weight rows, so neighbours share every cache line, and
		// with neighbours on different XCDs each line crossed the L2 boundary twice.
		const int b = (int)blockIdx.x - blocks_w;
		const int rows_x = (px.M + 31) / 32, total = cols_x * rows_x;
		const int x = b & 7, q = total >> 3, r = total & 7;
		const int idx = x * q + min(x, r) + (b >> 3);
		sgemm_skinny_body<2, false>(px, idx / rows_x, idx % rows_x, lds);
		return;
	}
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lrow = lane & 31, g = lane >> 5;
	if (blocks_w * 4 < tiles_w) {
		// so many tiles of dW that eight per workgroup still give every CU several workgroups: a whole-K tile per wavefront,
		// no exchange and no barrier (4096 x 4096 weights at batch 32: 58 -> 36 us for the pair)
		const int tile = (int)blockIdx.x * 8 + wave;
		if (tile < tiles_w) sgemm_tn_wave_tile_lines(pw, tile, lds + wave * SLAB);
		return;
	}
	const int slot = wave & 3, khalf = wave >> 2;
	const int tile = (int)blockIdx.x * 4 + slot;
	const bool active = tile < tiles_w;
	const int k_mid = min(pw.K, (((pw.K + 1) / 2 + 31) / 32) * 32);  // whole batches of 32 k in the lower half
	v16f acc;
#pragma unroll
	for (int r = 0; r < 16; r++) acc[r] = 0.0f;
	float asum = 0.0f;
	if (active) sgemm_tn_tile_lines_partial(pw, tile, khalf ? k_mid : 0, khalf ? pw.K : k_mid, lds + wave * SLAB, acc, asum);
	asum += __shfl_xor(asum, 32, 64);
	float* sums = lds + 4 * 16 * 64;
	__syncthreads();  // the slabs are no longer read
	if (khalf == 1) {
#pragma unroll
		for (int r = 0; r < 16; r++) lds[(slot * 16 + r) * 64 + lane] = acc[r];
		if (g == 0) sums[slot * 32 + lrow] = asum;
	}
	__syncthreads();
	if (khalf != 0 || !active) return;
	const int tiles_n = (pw.N + 31) / 32;
	const int m0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
	const int n = n0 + lrow;
	if (n < pw.N) {
		// register 4q + e of lane (lrow, g): row 8q + 4g + e, column lrow
#pragma unroll
		for (int r = 0; r < 16; r++) {
			const int row = m0 + (r >> 2) * 8 + g * 4 + (r & 3);
			if (row >= pw.M) continue;
			float* c = pw.C + (int64_t)row * pw.ldc + n;
			float out = pw.alpha * (acc[r] + lds[(slot * 16 + r) * 64 + lane]);
			if (pw.beta != 0.0f) out += pw.beta * *c;
			sgemm_store(pw, c, out);
		}
	}
	if (pw.rowsum != nullptr && n0 == 0 && g == 0 && m0 + lrow < pw.M) pw.rowsum[m0 + lrow] += asum + sums[slot * 32 + lrow];
}

// Both operands allow 16-byte loads along their contiguous dimension.
static bool operands_vec(const SProblem& p)
{
	return (p.lda & 3) == 0 && (p.ldb & 3) == 0 && (p.stride_a & 3) == 0 && (p.stride_b & 3) == 0 &&
	       ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0;
}

static int launch_direct(const SProblem& p, int tA, int tB, uint64_t batch)
{
	const dim3 grid((unsigned)(ceil_div(p.M, 32) * ceil_div(p.N, 32)), 1, (unsigned)batch), block(8 * 64);
	const bool vec = operands_vec(p);
	if (vec && p.K >= 512 && get_option(OPT_SGEMM_TILE) != 5) {  // at least two batches per wavefront
		set_kernel_name("sgemm_staged_32x32_w8");
		if (!tA && !tB) sgemm_staged_kernel<8, false, false><<<grid, block, 0, stream()>>>(p);
		if (!tA && tB) sgemm_staged_kernel<8, false, true><<<grid, block, 0, stream()>>>(p);
		if (tA && !tB) sgemm_staged_kernel<8, true, false><<<grid, block, 0, stream()>>>(p);
		if (tA && tB) sgemm_staged_kernel<8, true, true><<<grid, block, 0, stream()>>>(p);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	set_kernel_name("sgemm_direct_32x32_w8");
	if (!tA && !tB) sgemm_direct_kernel<8, false, false><<<grid, block, 0, stream()>>>(p);
	if (!tA && tB) sgemm_direct_kernel<8, false, true><<<grid, block, 0, stream()>>>(p);
	if (tA && !tB) sgemm_direct_kernel<8, true, false><<<grid, block, 0, stream()>>>(p);
	if (tA && tB) sgemm_direct_kernel<8, true, true><<<grid, block, 0, stream()>>>(p);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// K == 1: the rank-1 update C = alpha * a b^T + beta * C that l-ten uses to add the FC bias
// (l-ten/fully_connected.cpp:165).
__global__ __launch_bounds__(256) void sgemm_rank1_kernel(SProblem p, int tA, int tB)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= (int64_t)p.M * p.N) return;
	const int m = (int)(idx / p.N), n = (int)(idx % p.N);
	const float a = tA ? p.A[m] : p.A[(int64_t)m * p.lda];
	const float b = tB ? p.B[(int64_t)n * p.ldb] : p.B[n];
	float* c = p.C + (int64_t)m * p.ldc + n;
	float v = p.alpha * (a * b);
	if (p.beta != 0.0f) v += p.beta * *c;
	*c = v;
}

// The same, four columns per thread: N and ldc multiples of 4, C on a 16-byte boundary, b contiguous (tB == 0).
__global__ __launch_bounds__(256) void sgemm_rank1_vec4_kernel(SProblem p, int tA)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	const int n4 = p.N / 4;
	if (idx >= (int64_t)p.M * n4) return;
	const int m = (int)(idx / n4), n = (int)(idx - (int64_t)m * n4) * 4;
	const float a = tA ? p.A[m] : p.A[(int64_t)m * p.lda];
	const float4 b = *reinterpret_cast<const float4*>(p.B + n);
	float4* c = reinterpret_cast<float4*>(p.C + (int64_t)m * p.ldc + n);
	float4 v = make_float4(p.alpha * (a * b.x), p.alpha * (a * b.y), p.alpha * (a * b.z), p.alpha * (a * b.w));
	if (p.beta != 0.0f) {
		const float4 o = *c;
		v.x += p.beta * o.x; v.y += p.beta * o.y; v.z += p.beta * o.z; v.w += p.beta * o.w;
	}
	*c = v;
}

// C = alpha * A^T B + beta * C over a reduction of 2 to 8 rows (the weight gradient of a layer at a batch that small): a
// stream over C.  A thread takes four rows by four columns, so B's rows are read once per four rows of C; the products are
// added in the order of k.  N, ldb and ldc multiples of 4, B and C on 16-byte boundaries.
__global__ __launch_bounds__(256) void sgemm_tn_few_rows_kernel(SProblem p)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	const int n4 = p.N / 4, m4 = (p.M + 3) / 4;
	if (idx >= (int64_t)m4 * n4) return;
	const int m = (int)(idx / n4) * 4, n = (int)(idx % n4) * 4;
	float4 s[4];
#pragma unroll
	for (int r = 0; r < 4; r++) s[r] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	for (int k = 0; k < p.K; k++) {
		const float4 b = *reinterpret_cast<const float4*>(p.B + (int64_t)k * p.ldb + n);
		const float* a = p.A + (int64_t)k * p.lda + m;
#pragma unroll
		for (int r = 0; r < 4; r++) {
			const float ar = m + r < p.M ? a[r] : 0.0f;
			s[r].x += ar * b.x; s[r].y += ar * b.y; s[r].z += ar * b.z; s[r].w += ar * b.w;
		}
	}
#pragma unroll
	for (int r = 0; r < 4; r++) {
		if (m + r >= p.M) break;
		float4* c = reinterpret_cast<float4*>(p.C + (int64_t)(m + r) * p.ldc + n);
		float4 v = make_float4(p.alpha * s[r].x, p.alpha * s[r].y, p.alpha * s[r].z, p.alpha * s[r].w);
		if (p.beta != 0.0f) {
			const float4 o = *c;
			v.x += p.beta * o.x; v.y += p.beta * o.y; v.z += p.beta * o.z; v.w += p.beta * o.w;
		}
		*c = v;
	}
}

// M == 1 with B not transposed: c[n] = alpha * sum_k a[k] B[k][n] + beta * c[n] — the column sum that
// l-ten uses for the bias gradient with a = ones (l-ten/backprop.cpp:2267) and the two products of a GRU time
// step (l-ten/gru.cpp:267-268).  A workgroup takes COLS columns and cuts K into SLICES slices, one thread per
// (column, slice) with eight loads in flight; the slices are combined in slice order.  A null A stands for a
// vector of ones, so the bias_multiplier tensor of l-ten's FullyConnected is never needed on the device.
// Two shapes: 64 columns x 4 slices when the columns alone give every CU a workgroup, else 16 x 64 (rows
// are then read in 64-byte pieces, but four times as many workgroups share a long K).  blockIdx.z counts the problems
// of a strided batch (the x U and h W products of one GRU time step, l-ten/gru.cpp:358-361, are a batch of two when
// the input and hidden sizes agree): one launch for all of them.
template <int COLS, int SLICES>
__global__ __launch_bounds__(COLS* SLICES) void sgemm_rowvec_kernel(SProblem p, int tA)
{
	__shared__ float part[SLICES][COLS];
	const int tx = threadIdx.x % COLS, ty = threadIdx.x / COLS;
	// Consecutive workgroups go round-robin to the eight XCDs; XCD x takes a contiguous run of column blocks, so that
	// neighbours, which share the cache lines of every row of B (a block reads 64-byte pieces), meet in one L2: with
	// neighbours on different XCDs the matrix occupies the L2s twice and a step's two weight matrices no longer fit.
	const int nblk = gridDim.x, bx = blockIdx.x & 7, bq = nblk >> 3, br = nblk & 7;
	const int blk = bx * bq + min(bx, br) + ((int)blockIdx.x >> 3);
	const int n = blk * COLS + tx;
	const float* const A = p.A == nullptr ? nullptr : p.A + (int64_t)blockIdx.z * p.stride_a;
	const float* const B = p.B + (int64_t)blockIdx.z * p.stride_b;
	float* const C = p.C + (int64_t)blockIdx.z * p.stride_c;
	float s = 0.0f;
	if (n < p.N) {
		auto a_at = [&](int k) { return A == nullptr ? 1.0f : (tA ? A[(int64_t)k * p.lda] : A[k]); };
		const float* bcol = B + n;
		int k = ty;
		for (; k + 7 * SLICES < p.K; k += 8 * SLICES) {
			float bv[8], av[8];
#pragma unroll
			for (int u = 0; u < 8; u++) {
				bv[u] = bcol[(int64_t)(k + u * SLICES) * p.ldb];
				av[u] = a_at(k + u * SLICES);
			}
#pragma unroll
			for (int u = 0; u < 8; u++) s = fmaf(av[u], bv[u], s);
		}
		for (; k < p.K; k += SLICES) s = fmaf(a_at(k), bcol[(int64_t)k * p.ldb], s);
	}
	part[ty][tx] = s;
	__syncthreads();
	if (ty == 0 && n < p.N) {
		float v = part[0][tx];
#pragma unroll
		for (int q = 1; q < SLICES; q++) v += part[q][tx];
		v *= p.alpha;
		if (p.beta != 0.0f) v += p.beta * C[n];
		C[n] = v;
	}
}

static void launch_rowvec(const SProblem& p, int tA, uint64_t batch)
{
	set_kernel_name(batch > 1 ? "sgemm_rowvec_batched" : "sgemm_rowvec");
	if (ceil_div(p.N, 64) * batch >= 256 || p.K < 128)
		sgemm_rowvec_kernel<64, 4><<<dim3((unsigned)ceil_div(p.N, 64), 1, (unsigned)batch), dim3(256), 0, stream()>>>(p, tA);
	else
		sgemm_rowvec_kernel<16, 64><<<dim3((unsigned)ceil_div(p.N, 16), 1, (unsigned)batch), dim3(1024), 0, stream()>>>(p, tA);
}

template <int BM, int BN, int BK, int WM, int WN>
static int launch_sgemm(const SProblem& p, int tA, int tB, uint64_t batch, const char* name)
{
	const dim3 grid((unsigned)(ceil_div(p.M, BM) * ceil_div(p.N, BN)), 1, (unsigned)batch);
	const dim3 block(WM * WN * 64);
	set_kernel_name(name);
	if (!tA && !tB) sgemm_kernel<BM, BN, BK, WM, WN, false, false><<<grid, block, 0, stream()>>>(p);
	if (!tA && tB) sgemm_kernel<BM, BN, BK, WM, WN, false, true><<<grid, block, 0, stream()>>>(p);
	if (tA && !tB) sgemm_kernel<BM, BN, BK, WM, WN, true, false><<<grid, block, 0, stream()>>>(p);
	if (tA && tB) sgemm_kernel<BM, BN, BK, WM, WN, true, true><<<grid, block, 0, stream()>>>(p);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// C = alpha * (partial[0] + partial[1] + ...) + beta * C (+ bias per column), the partial matrices [parts][M][N] added in
// index order
__global__ __launch_bounds__(256) void sgemm_add_partials_kernel(const float* __restrict__ partial, int parts, int M, int N, float alpha, float beta,
                                                                 float* __restrict__ C, int64_t ldc, const float* __restrict__ bias)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x, count = (int64_t)M * N;
	if (idx >= count) return;
	// (the loads of 16 slices in flight at a time: one load per addition took 64 memory latencies for 64 slices, 15 us for a
	// 16 x 128 output)
	float sum = 0.0f;
	int s = 0;
	for (; s + 16 <= parts; s += 16) {
		float v[16];
#pragma unroll
		for (int j = 0; j < 16; j++) v[j] = partial[(int64_t)(s + j) * count + idx];
#pragma unroll
		for (int j = 0; j < 16; j++) sum += v[j];
	}
	if (s + 8 <= parts) {
		float v[8];
#pragma unroll
		for (int j = 0; j < 8; j++) v[j] = partial[(int64_t)(s + j) * count + idx];
#pragma unroll
		for (int j = 0; j < 8; j++) sum += v[j];
		s += 8;
	}
	for (; s < parts; s++) sum += partial[(int64_t)s * count + idx];
	const int64_t n = idx % N;
	float* c = C + (idx / N) * ldc + n;
	const float v = beta == 0.0f ? alpha * sum : alpha * sum + beta * *c;
	*c = bias ? v + bias[n] : v;
}

// dst[64][cols]: the first `rows` rows of src (leading dimension ld), zeros below
__global__ __launch_bounds__(256) void sgemm_pad_k_rows_kernel(const float* __restrict__ src, int64_t ld, int rows, int cols, float* __restrict__ dst)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one float4
	const int c4 = cols / 4;
	if (idx >= (int64_t)64 * c4) return;
	const int r = (int)(idx / c4), c = (int)(idx - (int64_t)r * c4) * 4;
	float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	if (r < rows) v = *reinterpret_cast<const float4*>(src + r * ld + c);
	reinterpret_cast<float4*>(dst)[idx] = v;
}

// dst[rows][64]: the first `cols` columns of src's rows (leading dimension ld), zeros behind them
__global__ __launch_bounds__(256) void sgemm_pad_k_cols_kernel(const float* __restrict__ src, int64_t ld, int64_t rows, int cols, float* __restrict__ dst)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one element
	if (idx >= rows * 64) return;
	const int64_t r = idx >> 6;
	const int c = (int)(idx & 63);
	dst[idx] = c < cols ? src[r * ld + c] : 0.0f;
}

int sgemm_run(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, float alpha, const float* A, uint64_t lda,
              int64_t stride_a, const float* B, uint64_t ldb, int64_t stride_b, float beta, float* C, uint64_t ldc,
              int64_t stride_c, uint64_t batch, const float* bias, float* rowsum, bool* rowsum_done, float* relu_out = nullptr,
              const float* relu_in = nullptr, bool* relu_done = nullptr)
{
	if (rowsum_done) *rowsum_done = false;
	if (relu_done) *relu_done = false;
	if (M == 0 || N == 0 || batch == 0) return 0;
	LTEN_HIP_REQUIRE(C != nullptr, "sgemm: C is null");
	LTEN_HIP_REQUIRE(K == 0 || (A != nullptr && B != nullptr), "sgemm: null operand");
	LTEN_HIP_REQUIRE(M < (1ull << 31) && N < (1ull << 31) && K < (1ull << 31) && batch < 65536, "sgemm: dimension too large");
	LTEN_HIP_REQUIRE(lda >= (tA ? M : K) && ldb >= (tB ? K : N) && ldc >= N, "sgemm: leading dimension smaller than the row");
	if (batch > 1 && !tA && stride_b == 0 && stride_a == (int64_t)(M * lda) && stride_c == (int64_t)(M * ldc) && batch * M < (1ull << 31) && rowsum == nullptr &&
	    relu_done == nullptr) {
		// A stack of matrices against one shared matrix, the stack's rows one behind the other in A and in C: one product
		// with batch * M rows (1024 x (16 x 128) against 128 x 128 is 16384 x 128 x 128, not 1024 products of 16 rows).
		return sgemm_run(0, tB, batch * M, N, K, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc, 0, 1, bias, nullptr, nullptr);
	}
	if (batch > 1 && stride_c == 0 && tA && !tB && bias == nullptr && stride_a == (int64_t)(K * lda) && stride_b == (int64_t)(K * ldb) &&
	    batch * K < (1ull << 31)) {
		// The problems' operands lie one behind the other along the reduction (the gradient of a matrix that a stack of
		// matrices was multiplied by: dB = sum over the stack of A_i^T dC_i, l-ten/backprop.cpp:533-585): one product with
		// batch * K rows to reduce over, instead of batch launches that each add to C.
		return sgemm_run(1, 0, M, N, batch * K, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc, 0, 1, nullptr, nullptr, nullptr);
	}
	if (batch > 1 && stride_c == 0) {
		// every problem writes the same C: run them one after another so the sum has one fixed order
		for (uint64_t b = 0; b < batch; b++) {
			int rc = sgemm_run(tA, tB, M, N, K, alpha, A + b * stride_a, lda, 0, B + b * stride_b, ldb, 0,
			                   (b == 0) ? beta : 1.0f, C, ldc, 0, 1, bias && b == 0 ? bias : nullptr, nullptr, nullptr);
			if (rc) return rc;
		}
		return 0;
	}
	// A^T B over a reduction of fewer than 64 rows into a large output (the weight gradient of a wide layer at a batch of
	// 32: 4096 x 25088 x 32) is bound by writing C, which the 32 x 32 kernels below do at 1.5 TB/s (100 000 workgroups of
	// eight wavefronts for one k-step each); the direct-to-LDS tiles want 64 rows at least, so the operands are copied into
	// 64 rows, the rest zero, in memory the library owns (7 MB against the 411 MB of C: 279 us before).
	// (2 to 8 rows: the stream over C below, 4096 x 25088 x 4 at the rate a fill reaches)
	if (get_option(OPT_SGEMM_TILE) == 0 && tA && !tB && batch == 1 && bias == nullptr && relu_done == nullptr && K >= 2 && K <= 8 && N % 4 == 0 && ldb % 4 == 0 &&
	    ldc % 4 == 0 && ((reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C)) & 15) == 0 && M * N >= (1u << 18) && M < (1ull << 31) && N < (1ull << 31)) {
		SProblem pf = {};
		pf.A = A; pf.B = B; pf.C = C;
		pf.lda = (int64_t)lda; pf.ldb = (int64_t)ldb; pf.ldc = (int64_t)ldc;
		pf.M = (int)M; pf.N = (int)N; pf.K = (int)K;
		pf.alpha = alpha; pf.beta = beta;
		set_kernel_name("sgemm_tn_few_rows");
		sgemm_tn_few_rows_kernel<<<dim3((unsigned)ceil_div(ceil_div(M, 4) * (N / 4), 256)), dim3(256), 0, stream()>>>(pf);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	if (get_option(OPT_SGEMM_TILE) == 0 && tA && !tB && batch == 1 && bias == nullptr && relu_done == nullptr && K >= 2 && K < 64 && M % 4 == 0 && N % 4 == 0 &&
	    lda % 4 == 0 && ldb % 4 == 0 && ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 &&
	    ceil_div(M, 128) * ceil_div(N, 128) >= 512) {
		float* rows64 = static_cast<float*>(library_scratch(64 * (M + N) * sizeof(float)));
		if (rows64 != nullptr) {
			sgemm_pad_k_rows_kernel<<<dim3((unsigned)ceil_div(16 * M, 256)), dim3(256), 0, stream()>>>(A, (int64_t)lda, (int)K, (int)M, rows64);
			sgemm_pad_k_rows_kernel<<<dim3((unsigned)ceil_div(16 * N, 256)), dim3(256), 0, stream()>>>(B, (int64_t)ldb, (int)K, (int)N, rows64 + 64 * M);
			LTEN_HIP_LAUNCH_CHECK();
			return sgemm_run(1, 0, M, N, 64, alpha, rows64, M, 0, rows64 + 64 * M, N, 0, beta, C, ldc, 0, 1, nullptr, nullptr, nullptr);
		}
	}
	// The same for A B and A B^T over 9 to 63 columns of A (a layer of that many inputs or outputs against a large batch: 12288
	// x 3072 x 48 ran 109 us on the 32 x 32 kernel): operands that are contiguous along K are copied into rows of 64.
	if (get_option(OPT_SGEMM_TILE) == 0 && !tA && batch == 1 && bias == nullptr && relu_done == nullptr && K > 8 && K < 64 && M > 64 && N > 64 &&
	    (tB || (N % 4 == 0 && ldb % 4 == 0 && (reinterpret_cast<uintptr_t>(B) & 15) == 0)) && ceil_div(M, 128) * ceil_div(N, 128) >= 512 && M < (1ull << 25) && N < (1ull << 25)) {  // (below 512 tiles the two copies cost what the tiles gain)
		float* a64 = static_cast<float*>(library_scratch(64 * (M + N) * sizeof(float)));
		if (a64 != nullptr) {
			float* b64 = a64 + 64 * M;
			sgemm_pad_k_cols_kernel<<<dim3((unsigned)ceil_div(64 * M, 256)), dim3(256), 0, stream()>>>(A, (int64_t)lda, (int64_t)M, (int)K, a64);
			if (tB) sgemm_pad_k_cols_kernel<<<dim3((unsigned)ceil_div(64 * N, 256)), dim3(256), 0, stream()>>>(B, (int64_t)ldb, (int64_t)N, (int)K, b64);
			else sgemm_pad_k_rows_kernel<<<dim3((unsigned)ceil_div(16 * N, 256)), dim3(256), 0, stream()>>>(B, (int64_t)ldb, (int)K, (int)N, b64);
			LTEN_HIP_LAUNCH_CHECK();
			return sgemm_run(0, tB, M, N, 64, alpha, a64, 64, 0, b64, tB ? 64 : N, 0, beta, C, ldc, 0, 1, nullptr, nullptr, nullptr);
		}
	}
	// A long reduction into a small output (the weight gradient of a small layer over a large batch: 128 x 128 x 16384)
	// gives the kernels below a handful of workgroups that each walk all of K: 114 us where the operands' 17 MB take 5.
	// K is cut into up to 64 slices (of 512 or more) that run as one strided batch into partial matrices (in memory the library owns),
	// which a second launch adds up in the order of the slices, so the result does not depend on timing.
	// (Not where the weight-streaming kernels below take the product: few rows against a long or wide weight matrix,
	// l-ten's 5760 -> 50 layer at batch 64, is their shape and cuts K over a workgroup's wavefronts already; from 128 rows
	// and a K of 8192 on the split is ahead of them: 384 x 384 x 16384 NT 97 -> 55 us, 128 x 256 x 8192 31 -> 20 us.)
	// (the NN streaming kernel wants more than 16 rows, a single row has the row-vector kernel: 2 to 16 rows against a long K
	// had neither and walked K on 32 workgroups, 4 x 1024 x 32000 in 202 us)
	// (up to 16 rows from K = 3072 on: the slices then run as a batch on the same streaming kernel, 1 x 4096 -> 1000 10.2 -> 6.6 us)
	const bool few_columns = K >= (M <= 16 ? 3072 : 8192) && ceil_div(N, 16) * ceil_div(M, 32) < (M <= 16 ? 128 : 256);  // (their workgroups, one per 16 columns, leave half of the CUs idle)
	const bool streams = (M < 128 || K < 8192) && ((!tA && tB && K % 4 == 0 && !few_columns) || (!tA && !tB && N >= 512 && (M == 1 || (M > 16 && !few_columns))));
	const bool small_out = !streams && K >= 1536 && ceil_div(M, 32) * ceil_div(N, 32) <= 256;
	// The same for outputs of 65 to 255 tiles of 64 x 64 under a reduction of 4096 or more: the direct-to-LDS tiles run at
	// their rate from about 512 workgroups on, so K is cut until the slices give that many (256 x 2304 x 6272, 144 tiles:
	// 104 us whole, 98 in two slices, 75 + 4 in four; 768 x 768 x 8192: 134 -> 96 + 4 us; 512 x 1024 x 8192, which the
	// weight-streaming kernels took at 104-133 us: 69 + 4 us).
	const uint64_t tiles64_all = ceil_div(M, 64) * ceil_div(N, 64);
	const bool mid_out = M >= 128 && N >= 128 && tiles64_all > 64 && tiles64_all < 256 && K >= 4096 && lda % 4 == 0 && ldb % 4 == 0 &&
	                     ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 && (tA ? M % 4 == 0 : true) && (tB ? true : N % 4 == 0);
	// A small stack of such products (matmul's gradient for a stack of tall matrices: 2 x (32 x 512 x 25088) TN took 174 us as
	// one batch of K-walking workgroups): one after the other, each split, 46 us; 8 x (16 x 16 x 65536) 442 -> 102 us.  With
	// more than 64 tiles of 32 x 32 in the stack, or a shorter K, the one batch is ahead (8 x (128 x 128 x 8192): 64 against 89 us).
	if (get_option(OPT_SGEMM_TILE) == 0 && batch > 1 && batch <= 8 && stride_c != 0 && bias == nullptr && K >= 8192 && small_out &&
	    ceil_div(M, 32) * ceil_div(N, 32) * batch <= 64) {
		for (uint64_t b = 0; b < batch; b++)
			if (int rc = sgemm_run(tA, tB, M, N, K, alpha, A + (int64_t)b * stride_a, lda, 0, B + (int64_t)b * stride_b, ldb, 0, beta, C + (int64_t)b * stride_c, ldc, 0, 1,
			                       nullptr, nullptr, nullptr))
				return rc;
		return 0;
	}
	// (a bias per column, FullyConnected's, rides on the launch that adds the slices)
	if (get_option(OPT_SGEMM_TILE) == 0 && batch == 1 && (small_out || mid_out)) {
		const uint64_t tiles32 = ceil_div(M, 32) * ceil_div(N, 32);
		uint64_t slices;
		if (small_out) {
			slices = std::min<uint64_t>(64, std::max<uint64_t>(2, 1024 / tiles32));  // (more slices were no faster: 64 x 64 x 65536 36 us with 64, 51 us with 128)
			// (slices of 512 or more; of 256 or more from K = 4096 on, where the slices then fill the direct-to-LDS 64 x 64 tiles:
			// 192 x 192 x 6144 in 12 slices 18.4 us, in 24 12.5; 128 x 128 x 16384 in 32 15.8, in 64 13.4; 1000 x 48 x 4096 14.4 -> 11.2)
			slices = std::max<uint64_t>(2, std::min<uint64_t>(slices, K / (K >= 4096 ? 256 : 512)));
			// (a count that divides K's steps of 32, if one is near: what the slices leave over costs a launch of its own,
			// 7 of the 26 us of 384 x 48 x 8192 in ten slices of 800)
			for (uint64_t s = slices; s > slices / 2 + 1 && s > 2; s--)
				if ((K / 32) % s == 0) {
					slices = s;
					break;
				}
		} else {
			slices = 2;
			while (tiles64_all * slices < 512 && slices < 16 && K / (slices * 2) >= 1024) slices *= 2;
		}
		const uint64_t kc = (K / slices) & ~31ull, rest = K - slices * kc, parts = slices + (rest != 0 ? 1 : 0);
		float* partial = kc >= 256 ? static_cast<float*>(library_scratch(parts * M * N * sizeof(float))) : nullptr;
		if (partial != nullptr) {
			// (what the slices leave over can be long enough to be split itself: its partial matrices go behind these)
			LibraryScratchHold hold(parts * M * N * sizeof(float));
			int rc = sgemm_run(tA, tB, M, N, kc, 1.0f, A, lda, (int64_t)(tA ? kc * lda : kc), B, ldb, (int64_t)(tB ? kc : kc * ldb), 0.0f, partial, N,
			                   (int64_t)(M * N), slices, nullptr, nullptr, nullptr);
			if (rc) return rc;
			if (rest != 0) {
				rc = sgemm_run(tA, tB, M, N, rest, 1.0f, A + (tA ? slices * kc * lda : slices * kc), lda, 0, B + (tB ? slices * kc : slices * kc * ldb), ldb, 0,
				               0.0f, partial + slices * M * N, N, 0, 1, nullptr, nullptr, nullptr);
				if (rc) return rc;
			}
			set_kernel_name("sgemm_split_k");
			sgemm_add_partials_kernel<<<dim3((unsigned)ceil_div(M * N, 256)), dim3(256), 0, stream()>>>(partial, (int)parts, (int)M, (int)N, alpha, beta, C, (int64_t)ldc, bias);
			LTEN_HIP_LAUNCH_CHECK();
			return 0;
		}
	}
	SProblem p;
	p.A = A; p.B = B; p.C = C; p.bias = bias; p.rowsum = nullptr; p.relu_out = nullptr; p.relu_in = nullptr;
	// the relu pieces ride on the kernels whose epilogue goes through sgemm_store; elsewhere the caller launches them
	const bool want_relu = relu_done != nullptr && batch == 1 && (relu_out != nullptr || relu_in != nullptr);
	p.lda = (int64_t)lda; p.ldb = (int64_t)ldb; p.ldc = (int64_t)ldc;
	p.stride_a = stride_a; p.stride_b = stride_b; p.stride_c = stride_c;
	p.M = (int)M; p.N = (int)N; p.K = (int)K;
	p.alpha = alpha; p.beta = beta;

	const int force = get_option(OPT_SGEMM_TILE);
	if (force == 0 && batch == 1 && bias == nullptr && K == 1) {
		set_kernel_name("sgemm_rank1");
		if (!tB && N % 4 == 0 && ldc % 4 == 0 && ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 && M * N >= (1u << 16))
			sgemm_rank1_vec4_kernel<<<dim3((unsigned)ceil_div(M * (N / 4), 256)), dim3(256), 0, stream()>>>(p, tA);
		else sgemm_rank1_kernel<<<dim3((unsigned)ceil_div(M * N, 256)), dim3(256), 0, stream()>>>(p, tA, tB);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	if (force == 0 && bias == nullptr && M == 1 && !tB) {
		launch_rowvec(p, tA, batch);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	// FullyConnected forward with few activation rows: 16 columns of the weights per workgroup, and for more than 32
	// rows one workgroup per block of 32 rows as well (the weights then come from the L2 for all but the first), while
	// that gives at most a few workgroups per CU: 128 rows against a 1024-wide layer are 256 tiles of 32 x 16 where the
	// 32 x 32 tiles of the general small-GEMM kernels would occupy half of the CUs.
	// A classifier head (a few output columns) takes the same kernel: one column block, K cut over eight wavefronts.
	// (a strided batch of such products with at most 16 rows each, the slices of a split reduction among them, runs on
	// the grid's planes)
	const bool skinny_batch = batch > 1 && batch < 65536 && M <= 16 && bias == nullptr && stride_c != 0 && stride_a % 4 == 0 && stride_b % 4 == 0;
	if (force == 0 && !tA && tB && K >= 256 && K % 4 == 0 && (batch == 1 || skinny_batch) && operands_vec(p) &&
	    (M <= 32 || ceil_div(M, 32) * ceil_div(N, 16) <= 1024)) {
		// few column blocks (a classifier head): blocks of 16 rows, twice the workgroups
		const bool rows16 = M <= 16 || ceil_div(N, 16) * ceil_div(M, 32) < 64;
		set_kernel_name(rows16 ? "sgemm_skinny_nt_16x16" : "sgemm_skinny_nt_32x16");
		if (want_relu) { p.relu_out = relu_out; p.relu_in = relu_in; *relu_done = true; }
		const dim3 grid((unsigned)ceil_div(N, 16), (unsigned)(rows16 ? ceil_div(M, 16) : ceil_div(M, 32)), (unsigned)batch);
		if (rows16) sgemm_skinny_nt_kernel<1><<<grid, dim3(512), 0, stream()>>>(p);
		else sgemm_skinny_nt_kernel<2><<<grid, dim3(512), 0, stream()>>>(p);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	// The NN product with few rows (the data gradient of such a layer) on the same tiles.
	if (force == 0 && !tA && !tB && N >= 512 && N % 4 == 0 && K >= 256 && K % 4 == 0 && batch == 1 && operands_vec(p) && M > 16 &&
	    ceil_div(M, 32) * ceil_div(N, 16) <= 1024) {
		set_kernel_name("sgemm_skinny_nn_32x16");
		if (want_relu) { p.relu_out = relu_out; p.relu_in = relu_in; *relu_done = true; }
		sgemm_skinny_nn_kernel<2><<<dim3((unsigned)ceil_div(N, 16), (unsigned)ceil_div(M, 32)), dim3(512), 0, stream()>>>(p);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	const uint64_t tiles64 = ceil_div(M, 64) * ceil_div(N, 64) * batch;
	const uint64_t tiles128 = ceil_div(M, 128) * ceil_div(N, 128) * batch;
	int choice = force;
	if (choice >= 10) {  // a direct-to-LDS tile by number; falls through to the heuristic when the problem does not fit
		if (sgemm_fast_dispatch(p, tA, tB, batch, choice) == 0) return 0;
		choice = 0;
	}
	// Products whose 128 x 128 tiles would not give every CU a workgroup while 64 x 64 tiles fill half of them or more (a
	// FullyConnected layer at a batch of 256 to 768 against a 4096-wide layer: 512 x 4096 x 4096 forward in 132 us
	// instead of 240, the time of batch 1024; its data and weight gradients 130 instead of 237 us; 1024^3 in any layout
	// 22 instead of 37 us)
	// (and products with a side of at most 64, which would leave half or more of every larger tile empty: a batch of 96
	// products 512 x 64 x 512 took 125 us on 256 x 256 tiles)
	const bool t64 = (tiles128 < 256 || M <= 64 || N <= 64) && tiles64 >= 128;
	// (a short K, 64 to 255 in whole steps of 32, only with many tiles: the products of a batch of attention heads, or an
	// outer-product-like update; 96 x (512 x 512 x 64): 78-91 us on the 32 x 32 kernel, 45 us here; 4096 x 4096 x 64:
	// 52-58 and 28 us; with 96 tiles of 128 x 128 the two are level)
	// (measured again over batches of small products: at K = 64 the 128 x 128 tiles are ahead from 192 of them on, 16 x (512 x
	// 512 x 64) 17 -> 9 us, 96 x (256 x 256 x 64) 24 -> 13 us, 2048 x 2048 x 64 17 -> 9 us, and behind with 64, where the 32 x
	// 32 kernel stays; from K = 96 on the 64 x 64 tiles from 256 of them on: 8 x (512 x 512 x 128) 13 -> 10 us, 384 x (128 x 64 x
	// 128) 22 -> 16 us, 2048 x 1024 x 96 11 -> 9 us)
	const bool many128 = tiles128 >= 192 && M > 64 && N > 64;
	const bool short_k = K >= 64 && K < 256 && K % 32 == 0 && (tiles128 >= 512 || many128 || (K >= 96 && tiles64 >= 256));
	if (choice == 0 && (tiles128 >= 128 || t64) && ((K >= 256 && (K % 32 == 0 || K >= 512)) || short_k)) {
		// large problems: 256 x 256 tiles when they fill the chip, else 128 x 128 (or 64 x 64, above).  The tiles walk K in
		// steps of 32: what is left over is added by a second, general launch (beta = 1, no bias).
		const bool big = ceil_div(M, 256) * ceil_div(N, 256) * batch >= 192 && M >= 192 && N >= 192 && !short_k;
		const uint64_t k_main = K & ~31ull;
		p.K = (int)k_main;
		if (sgemm_fast_dispatch(p, tA, tB, batch, big ? 12 : (t64 && !(K < 96 && many128) ? 31 : 21)) == 0) {
			if (k_main == K) return 0;
			return sgemm_run(tA, tB, M, N, K - k_main, alpha, A + (tA ? k_main * lda : k_main), lda, stride_a,
			                 B + (tB ? k_main : k_main * ldb), ldb, stride_b, 1.0f, C, ldc, stride_c, batch, nullptr, nullptr, nullptr);
		}
		p.K = (int)K;
	}
	if (choice == 0) {
		// Few output tiles and a long K: the LDS-tiled kernels would leave most CUs idle while a handful of
		// workgroups walk K in sequence; the direct kernel cuts K across the wavefronts of a workgroup instead.
		// With 16-byte loads the 32x32 kernels stay ahead of the LDS-tiled ones at every size measured (1280^3: 74 vs
		// 80 us, 200 x 5000 x 700: 45 vs 44 us); without them while the tiles are few, except for NT products,
		// whose 4-byte loads along K they handle badly (1001 x 1003 x 1005: NN 55 vs 51 us, TN 40 vs 51, NT 83 vs 48).
		// Of the LDS-tiled kernels the 64 x 64 tile is ahead until the problem is large (2047 x 2049 x 513: 79 vs 103 us,
		// 6000 x 500 x 999: 89 vs 128 us; 4095^3: 1677 vs 1424 us).
		const uint64_t tiles32 = ceil_div(M, 32) * ceil_div(N, 32) * batch;
		const int lds_tiled = tiles128 >= 512 ? 1 : 2;
		if (operands_vec(p) && tiles32 < (1u << 20)) choice = 4;
		else if (!tA && tB) choice = tiles64 >= 64 ? lds_tiled : 4;
		else choice = tiles32 <= 1024 ? 4 : lds_tiled;
	}
	if (want_relu) { p.relu_out = relu_out; p.relu_in = relu_in; *relu_done = true; }
	switch (choice) {
	case 1: return launch_sgemm<128, 128, 16, 2, 2>(p, tA, tB, batch, "sgemm_128x128x16");
	case 2: return launch_sgemm<64, 64, 32, 2, 2>(p, tA, tB, batch, "sgemm_64x64x32");
	case 3: return launch_sgemm<32, 32, 32, 1, 1>(p, tA, tB, batch, "sgemm_32x32x32");
	default:
		if (rowsum != nullptr && rowsum_done != nullptr && batch == 1 && K != 0) {
			p.rowsum = rowsum;
			*rowsum_done = true;
		}
		return launch_direct(p, tA, tB, batch);
	}
}

// Whether sgemm_run sends a product without bias and batch (M x N x K, neither M, N nor K equal to 1) to the 32x32
// kernels: not large enough for the direct-to-LDS tiles (nor a short reduction over many of them), and few tiles or
// operands that allow 16-byte loads.
static bool takes_32x32(const SProblem& p, uint64_t M, uint64_t N, uint64_t K)
{
	if (K <= 1 || M <= 1) return false;
	const uint64_t tiles128 = ceil_div(M, 128) * ceil_div(N, 128);
	if (tiles128 >= 128 && K >= 256) return false;
	// the short reductions sgemm_run gives to the 128 x 128 tiles, where those are clearly ahead (the weight gradient of a
	// 4096-wide layer at a batch of 64: level; 128 x 8192 -> 8192, both gradients: 326 us with it there, 530 us without)
	if (K >= 64 && K < 256 && K % 32 == 0 && tiles128 >= 512 && (tiles128 >= 1024 || K >= 128)) return false;
	const uint64_t tiles32 = ceil_div(M, 32) * ceil_div(N, 32);
	return tiles32 <= 1024 || (operands_vec(p) && tiles32 < (1u << 20));
}

// The tile for a product with grouped columns and what it is expected to take, in us: the work of whole tiles at the rate
// measured for each size (256 x 256: 120 TFLOP/s, 128 x 128: 92, 64 x 64: 110), in proportion to the CUs the tiles fill.
double sgemm_grouped_columns_estimate(uint64_t M, uint64_t N, uint64_t K, int* variant)
{
	const int sizes[3] = { 256, 128, 64 }, variants[3] = { 12, 21, 31 };
	const double rates[3] = { 120e6, 92e6, 110e6 };
	double best = 0.0;
	for (int i = 0; i < 3; i++) {
		const uint64_t t = (uint64_t)sizes[i], tiles = ceil_div(M, t) * ceil_div(N, t);
		if (i == 0 && (M < 192 || N < 192)) continue;
		const double us = 2.0 * (double)(ceil_div(M, t) * t) * (double)(ceil_div(N, t) * t) * (double)K / (rates[i] * std::min(1.0, (double)tiles / 256.0));
		if (best == 0.0 || us < best) {
			best = us;
			if (variant) *variant = variants[i];
		}
	}
	return best;
}

int sgemm_grouped_columns(uint64_t M, uint64_t N, uint64_t K, const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t group,
                          int64_t group_stride, const float* row_bias)
{
	if (M == 0 || N == 0 || K < 64 || K % 32 != 0 || group == 0 || M >= (1ull << 31) || N >= (1ull << 31) || K >= (1ull << 31) || group >= (1ull << 31)) return -1;
	SProblem p = {};
	p.A = A; p.B = B; p.C = C;
	p.lda = (int64_t)lda; p.ldb = (int64_t)ldb; p.ldc = (int64_t)group;
	p.M = (int)M; p.N = (int)N; p.K = (int)K;
	p.alpha = 1.0f; p.beta = 0.0f;
	p.col_group = (int)group;
	p.col_group_stride = group_stride;
	p.row_bias = row_bias;
	int variant = 31;
	(void)sgemm_grouped_columns_estimate(M, N, K, &variant);
	return sgemm_fast_dispatch(p, 0, 0, 1, variant);
}

}  // namespace lten_hip

using namespace lten_hip;

extern "C" {

int lten_hip_sgemm(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, float alpha, const float* A, uint64_t lda,
                   const float* B, uint64_t ldb, float beta, float* C, uint64_t ldc)
{
	return sgemm_run(tA, tB, M, N, K, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc, 0, 1, nullptr, nullptr, nullptr);
}

int lten_hip_sgemm_strided_batched(int tA, int tB, uint64_t M, uint64_t N, uint64_t K, float alpha, const float* A,
                                   uint64_t lda, int64_t stride_a, const float* B, uint64_t ldb, int64_t stride_b,
                                   float beta, float* C, uint64_t ldc, int64_t stride_c, uint64_t batch)
{
	return sgemm_run(tA, tB, M, N, K, alpha, A, lda, stride_a, B, ldb, stride_b, beta, C, ldc, stride_c, batch, nullptr, nullptr, nullptr);
}

int lten_hip_fc_forward_f32(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W, const float* bias,
                            float* Y)
{
	// l-ten/fully_connected.cpp:150 (NT GEMM) and :165 (ones x bias, beta = 1) in one launch
	return sgemm_run(0, 1, M, out, in, 1.0f, X, in, 0, W, in, 0, 0.0f, Y, out, 0, 1, bias, nullptr, nullptr);
}

int lten_hip_fc_forward_relu_f32(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W, const float* bias,
                                 float* Y, float* Y_relu)
{
	LTEN_HIP_REQUIRE(Y_relu != nullptr || M * out == 0, "fc_forward_relu: Y_relu is null");
	bool relu_done = false;
	int rc = sgemm_run(0, 1, M, out, in, 1.0f, X, in, 0, W, in, 0, 0.0f, Y, out, 0, 1, bias, nullptr, nullptr, Y_relu, nullptr, &relu_done);
	// kernels without the fused store (the large direct-to-LDS tiles, the degenerate shapes): relu as a launch of its own
	if (!rc && !relu_done) rc = lten_hip_relu_f32(Y_relu, Y, M * out);
	return rc;
}

}  // extern "C"

static int fc_backward(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W, const float* dY,
                       const float* relu_input, float* dX, float* dW, float* db)
{
	int rc = 0;
	// Both products wanted, both of the kind the 32x32 kernels take (few tiles, or 16-byte loads possible; not one of
	// the degenerate shapes with a kernel of their own, not large enough for the direct-to-LDS tiles) and the batch
	// small enough that the weight-gradient product would not take the whole-line loads: one launch computes the two.
	// option "sgemm_tile" 7: the paired launch with the weight gradient's K cut over the wavefronts whatever the batch
	const int pair_opt = get_option(OPT_SGEMM_TILE);
	if (dX && dW && (pair_opt == 0 || pair_opt == 7) && M > 1 && M < 512 && out > 1 && out <= 8192 && in > 0) {
		SProblem px = {}, pw = {};
		px.A = dY; px.B = W; px.C = dX; px.lda = (int64_t)out; px.ldb = (int64_t)in; px.ldc = (int64_t)in;
		px.M = (int)M; px.N = (int)in; px.K = (int)out; px.alpha = 1.0f; px.beta = 0.0f;
		px.relu_in = relu_input;
		pw.A = dY; pw.B = X; pw.C = dW; pw.lda = (int64_t)out; pw.ldb = (int64_t)in; pw.ldc = (int64_t)in;
		pw.M = (int)out; pw.N = (int)in; pw.K = (int)M; pw.alpha = 1.0f; pw.beta = 0.0f;
		pw.rowsum = db;
		const uint64_t blocks_x = ceil_div(M, 32) * ceil_div(in, 32), blocks_w = ceil_div(out, 32) * ceil_div(in, 32);
		if (takes_32x32(px, M, in, out) && takes_32x32(pw, out, in, M) && blocks_x + blocks_w < (1u << 20)) {
			// dW: four tiles per workgroup (K cut in two over the wavefronts), eight whole-K tiles when that still leaves 2048 workgroups
			const uint64_t cols_x = ceil_div(in, 16), skinny_x = cols_x * ceil_div(M, 32), w4 = blocks_w >= 4096 ? ceil_div(blocks_w, 8) : ceil_div(blocks_w, 4);
			if (pair_opt == 0 && M > 1 && M <= 256 && blocks_w >= 256 && in >= 512 && in % 4 == 0 && out >= 256 && out % 4 == 0 &&
			    operands_vec(px) && operands_vec(pw) && skinny_x <= 1024) {
				set_kernel_name("sgemm_fc_backward_pair_wide");
				sgemm_fc_backward_pair_wide_kernel<<<dim3((unsigned)(w4 + skinny_x)), dim3(512), 0, stream()>>>(px, pw, (int)w4, (int)blocks_w, (int)cols_x);
			} else if (M <= 256 && blocks_w >= 256 && pair_opt == 0) {  // a short reduction and many tiles for dW: whole-K tiles per wavefront
				set_kernel_name("sgemm_fc_backward_pair_32x32_shortk");
				const dim3 grid((unsigned)(blocks_x + ceil_div(blocks_w, 8)));
				if (operands_vec(pw) && out % 4 == 0 && in % 4 == 0) sgemm_fc_backward_pair_shortk_kernel<true><<<grid, dim3(512), 0, stream()>>>(px, pw, (int)blocks_x);
				else sgemm_fc_backward_pair_shortk_kernel<false><<<grid, dim3(512), 0, stream()>>>(px, pw, (int)blocks_x);
			} else {
				set_kernel_name("sgemm_fc_backward_pair_32x32_w8");
				sgemm_fc_backward_pair_kernel<<<dim3((unsigned)(blocks_x + blocks_w)), dim3(512), 0, stream()>>>(px, pw, (int)blocks_x);
			}
			LTEN_HIP_LAUNCH_CHECK();
			return 0;
		}
	}
	// l-ten/backprop.cpp:2228  dX[M x in] = dY[M x out] W[out x in]
	if (dX) {
		bool relu_done = false;
		rc = sgemm_run(0, 0, M, in, out, 1.0f, dY, out, 0, W, in, 0, 0.0f, dX, in, 0, 1, nullptr, nullptr, nullptr, nullptr, relu_input,
		               relu_input ? &relu_done : nullptr);
		if (!rc && relu_input && !relu_done) rc = lten_hip_relu_backward_f32(dX, dX, relu_input, M * in);
	}
	// :2252  dW[out x in] = dY[M x out]^T X[M x in].  The rows of dY^T summed over the batch are the bias gradient
	// of :2267, so a kernel that can do it adds them into db on the way.
	bool db_done = false;
	if (!rc && dW) rc = sgemm_run(1, 0, out, in, M, 1.0f, dY, out, 0, X, in, 0, 0.0f, dW, in, 0, 1, nullptr, db, &db_done);
	// :2267  db[1 x out] += ones[1 x M] dY[M x out]; the ones vector is never materialised: a = 1 for every k
	if (!rc && db && !db_done && M != 0 && out != 0) {
		SProblem p = {};
		p.A = nullptr;  // a[k] = 1
		p.B = dY; p.C = db;
		p.ldb = (int64_t)out; p.ldc = (int64_t)out;
		p.M = 1; p.N = (int)out; p.K = (int)M;
		p.alpha = 1.0f; p.beta = 1.0f;
		launch_rowvec(p, 0, 1);
		LTEN_HIP_LAUNCH_CHECK();
	}
	return rc;
}

extern "C" {

int lten_hip_fc_backward_f32(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W, const float* dY,
                             float* dX, float* dW, float* db)
{
	return fc_backward(M, in, out, X, W, dY, nullptr, dX, dW, db);
}

int lten_hip_fc_backward_relu_f32(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W, const float* dY,
                                  const float* relu_input, float* dX, float* dW, float* db)
{
	LTEN_HIP_REQUIRE(relu_input != nullptr || dX == nullptr || M * in == 0, "fc_backward_relu: relu_input is null");
	return fc_backward(M, in, out, X, W, dY, relu_input, dX, dW, db);
}

int lten_hip_fc_backward_log_softmax_nll_loss_f32(uint64_t M, uint64_t in, uint64_t out, const float* X, const float* W, const float* logits,
                                                  const float* target, float alpha, float* log_probs, float* loss, float* dlogits,
                                                  const float* relu_input, float* dX, float* dW, float* db)
{
	LTEN_HIP_REQUIRE(loss != nullptr && M > 0, "fc_backward_log_softmax_nll_loss: null loss pointer or zero batch");
	LTEN_HIP_REQUIRE(out == 0 || (logits && target && log_probs && dlogits), "fc_backward_log_softmax_nll_loss: null pointer");
	const uint64_t blocks_x = ceil_div(M, 32) * ceil_div(in, 32), blocks_w = ceil_div(out, 32) * ceil_div(in, 32);
	if (dX && dW && X && W && get_option(OPT_SGEMM_TILE) == 0 && M > 1 && M < 512 && out > 1 && out <= 16 && M * out <= 4096 && in > 0 &&
	    blocks_w < 256) {
		SProblem px = {}, pw = {};
		px.A = dlogits; px.B = W; px.C = dX; px.lda = (int64_t)out; px.ldb = (int64_t)in; px.ldc = (int64_t)in;
		px.M = (int)M; px.N = (int)in; px.K = (int)out; px.alpha = 1.0f; px.beta = 0.0f;
		px.relu_in = relu_input;
		pw.A = dlogits; pw.B = X; pw.C = dW; pw.lda = (int64_t)out; pw.ldb = (int64_t)in; pw.ldc = (int64_t)in;
		pw.M = (int)out; pw.N = (int)in; pw.K = (int)M; pw.alpha = 1.0f; pw.beta = 0.0f;
		pw.rowsum = db;
		if (takes_32x32(px, M, in, out) && takes_32x32(pw, out, in, M) && blocks_x + blocks_w < (1u << 20)) {
			LossRows L = { (int)M, (int)out, logits, target, alpha, -1.0f / (float)M, log_probs, loss, dlogits };
			set_kernel_name("sgemm_fc_backward_pair_loss");
			sgemm_fc_backward_pair_loss_kernel<<<dim3((unsigned)(blocks_x + blocks_w)), dim3(512), 0, stream()>>>(px, pw, (int)blocks_x, L);
			LTEN_HIP_LAUNCH_CHECK();
			return 0;
		}
	}
	// the launches it stands for
	if (int rc = lten_hip_log_softmax_nll_loss_grad_f32(M, out, logits, target, alpha, log_probs, loss, dlogits)) return rc;
	return fc_backward(M, in, out, X, W, dlogits, relu_input, dX, dW, db);
}

}  // extern "C"
