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
	int64_t lda, ldb, ldc;
	int64_t stride_a, stride_b, stride_c;  // per blockIdx.z
	int M, N, K;
	float alpha, beta;
};

// Direct-to-LDS tiles for large aligned problems; returns -1 when the problem does not fit them.
int sgemm_fast_dispatch(const SProblem& p, int tA, int tB, uint64_t batch, int variant);

}  // namespace lten_hip
