// The problem descriptor of the fp32 GEMM kernels.
#pragma once

#include <cstdint>

namespace lten_hip {

// C[m][n] = alpha * sum_k op(A)[m][k] op(B)[k][n] + beta * C[m][n] (+ bias[n]), row-major.
// A[m][k] is at A[m*lda + k] (not transposed) or A[k*lda + m] (transposed); B[k][n] is at B[k*ldb + n]
// (not transposed) or B[n*ldb + k] (transposed).
struct SProblem {
	const float* A;
	const float* B;
	float* C;
	const float* bias;  // optional, added per output column n (FullyConnected bias), or null
	float* rowsum;      // optional: rowsum[m] += sum_k op(A)[m][k] (the FullyConnected bias gradient inside the
	                    // weight-gradient product); only the 32x32 kernels do it, for a single problem
	// Optional relu pieces of a training step folded into the store (single problems only; same indexing as C):
	float* relu_out;       // also receives max(C, 0): the activation next to the pre-activation (l-ten/layers.cpp:9-67)
	const float* relu_in;  // C = relu_in > 0 ? C : 0: relu_backward on the data gradient (l-ten/backprop.cpp:2282-2327)
	int64_t lda, ldb, ldc;
	int64_t stride_a, stride_b, stride_c;  // per blockIdx.z
	int M, N, K;
	float alpha, beta;
	// direct-to-LDS tiles only (set by their launcher): all tiles of a problem of the batch go to one XCD
	int problems_by_xcd = 0;
	// direct-to-LDS tiles only: the columns of C lie in groups of col_group, group g at C + g * col_group_stride and rows
	// ldc apart inside it (the output maps of a batch of images, [image][channel][pixel], as one matrix [channel][all pixels])
	int col_group = 0;
	int64_t col_group_stride = 0;
	const float* row_bias = nullptr;  // with col_group: added per row m (a convolution's bias per output channel), or null
};

// The last step of every epilogue that supports the relu pieces: c points into p.C (batch index 0).
__device__ __forceinline__ void sgemm_store(const SProblem& p, float* c, float out)
{
	if (p.relu_in != nullptr && !(p.relu_in[c - p.C] > 0)) out = 0.0f;
	*c = out;
	if (p.relu_out != nullptr) p.relu_out[c - p.C] = out > 0 ? out : 0.0f;
}

// Direct-to-LDS tiles for large aligned problems; returns -1 when the problem does not fit them.
int sgemm_fast_dispatch(const SProblem& p, int tA, int tB, uint64_t batch, int variant);
// C[m][(g, j)] = sum_k A[m][k] B[k][g * group + j] on the direct-to-LDS tiles (A row-major with K contiguous, B row-major
// with all N columns contiguous), column (g, j) stored at C + g * group_stride + m * group + j, plus row_bias[m] when that
// is not null; -1 when the tiles do not take the shapes.
double sgemm_grouped_columns_estimate(uint64_t M, uint64_t N, uint64_t K, int* variant);
int sgemm_grouped_columns(uint64_t M, uint64_t N, uint64_t K, const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t group,
                          int64_t group_stride, const float* row_bias);

}  // namespace lten_hip
