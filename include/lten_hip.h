/* lten_hip.h — C ABI of the MI355X (gfx950) GEMM hot path for light-tensor ("l-ten").
 *
 * Every entry point takes plain pointers and sizes.  Device pointers are raw HIP
 * device addresses (what lten_hip_alloc returns, or any hipMalloc'ed memory); the
 * caller owns every buffer and no call retains a pointer after it returns.  All work
 * is issued on one stream per process (the null stream unless lten_hip_set_stream is
 * called) and is stream ordered: kernels are asynchronous, lten_hip_copy_from_gpu and
 * lten_hip_sync are the synchronisation points — the model l-ten's GPU branches
 * already assume (l-ten/utils.cu:73-94 synchronous copies, default stream elsewhere).
 *
 * Return value: 0 on success, non-zero on failure with a message available from
 * lten_hip_last_error().  A C ABI cannot throw; the C++ glue turns a non-zero status
 * into LTEN_ERR, which is how l-ten reports failures (l-ten/error.h:78-93).
 *
 * Matrices are row-major, as every l-ten tensor is.
 */
#ifndef LTEN_HIP_H
#define LTEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Layout-identical to l-ten's QuantizationParams (l-ten/math_fns.h:12-16). */
typedef struct lten_hip_qparams {
	float   scale;
	uint8_t zero_point;
} lten_hip_qparams;

/* ------------------------------------------------------------------ context / errors */

/* Replaces the lazy cuBLAS/cuDNN handle creation of CUDA_globlas (l-ten/globals.h:89-123).
 * Selects `device`, checks that it is a gfx950 part. Idempotent. */
int lten_hip_init(int device);
/* Message of the last failing call on this thread ("" if none). */
const char* lten_hip_last_error(void);
/* Replaces GetDevice (l-ten/utils.h:41, l-ten/utils.cu:110-116). */
int lten_hip_get_device(int* device);
/* Routes all later work to `hip_stream` (a hipStream_t; NULL = the null stream), after waiting for the work
 * already issued on the stream it leaves (blocks that lten_hip_free returned to the pool while that work was pending
 * may be handed out again at once).  No counterpart in l-ten, which only ever uses the default stream. */
int lten_hip_set_stream(void* hip_stream);
/* Blocks until the stream is idle. l-ten's equivalent is the implicit sync of cudaMemcpy. */
int lten_hip_sync(void);

/* ------------------------------------------------------------------------- memory */

/* Replaces AllocateMemoryOnGPU / gpu_alloc (l-ten/utils.h:29,33; l-ten/utils.cu:8-28,30-58), memory pool included
 * (l-ten's default build serves GPU buffers from its power-of-two MemoryPool, l-ten/utils.cu:33-37,
 * l-ten/memorypool.h:142-173): sizes are rounded up to a power of two (to a multiple of 64 MB above 64 MB), freed
 * blocks are kept and handed out again without a wait — correct for work issued in order on the library's stream
 * (a caller that uses a block on a stream of its own must finish that work before it frees the block).  Up to 16 GB
 * stay cached; they go back to the driver when an allocation would otherwise fail or lten_hip_pool_release is called. */
int lten_hip_alloc(void** device_ptr, uint64_t size, int zero_memory);
/* Replaces FreeMemoryOnGPU / gpu_free (l-ten/utils.h:30,35; l-ten/utils.cu:60-71).  Freeing a block twice fails. */
int lten_hip_free(void* device_ptr);
/* Gives every cached block back to the driver (l-ten's MemoryPool frees its blocks only in its destructor,
 * l-ten/memorypool.h; a library has no such moment).  Blocks in use are not touched. */
int lten_hip_pool_release(void);
/* Replaces ZeroMemoryOnGPU (l-ten/utils.h:34; l-ten/utils.cu:49-52). */
int lten_hip_zero(void* device_ptr, size_t size);
/* Replace CopyDataToGPU / CopyDataFromGPU / GPUToGPUCopy (l-ten/utils.h:36-38; l-ten/utils.cu:73-108).
 * Host <-> device copies return after the data has arrived, as cudaMemcpy does. */
int lten_hip_copy_to_gpu(void* device_dst, const void* host_src, size_t size);
int lten_hip_copy_from_gpu(void* host_dst, const void* device_src, size_t size);
int lten_hip_copy_gpu_to_gpu(void* device_dst, const void* device_src, size_t size);

/* Replace gpu_fill<T> (l-ten/math_fns.h:180-181; l-ten/math_fns.cu:729-775). */
int lten_hip_fill_f32(float* device_ptr, uint64_t count, float value);
int lten_hip_fill_i32(int32_t* device_ptr, uint64_t count, int32_t value);
int lten_hip_fill_u8(uint8_t* device_ptr, uint64_t count, uint8_t value);

/* ----------------------------------------------------------------------- fp32 GEMM */

/* C[M x N] = alpha * op(A) * op(B) + beta * C, row-major with leading dimensions.
 * The contract of cpu_gemm<float> (l-ten/math_fns.h:18-19, l-ten/math_fns.cpp:1258) plus
 * lda/ldb/ldc; replaces every cublasSgemm site of l-ten's GPU branches
 * (l-ten/fully_connected.cpp:150,165; l-ten/conv2d.cpp:169; l-ten/md_array_cuda.h:513;
 * l-ten/backprop.cpp:562,580,2003,2024,2228,2252,2267).  beta == 0 overwrites C
 * (NaN/Inf in C are not propagated); A and B are never modified.  The K == 1
 * (bias rank-1 update) and M == 1 (bias-gradient column sum) shapes those sites use
 * are served by dedicated kernels.  A reduction of 1536 or more into a small output
 * (a weight gradient over a large batch), or of 4096 or more into one of up to 255 tiles
 * of 64 x 64, is cut into slices whose partial sums live in memory the library owns and
 * are added in a fixed order. */
int lten_hip_sgemm(int trans_a, int trans_b, uint64_t M, uint64_t N, uint64_t K, float alpha,
                   const float* A, uint64_t lda, const float* B, uint64_t ldb, float beta,
                   float* C, uint64_t ldc);

/* `batch` GEMMs with element strides between consecutive problems; a stride of 0
 * re-uses (broadcasts) that operand.  Serves the per-leading-index loop of
 * CUDA_MultiDimArray::matmul (l-ten/md_array_cuda.h:450-525) and matmul_backward
 * (l-ten/backprop.cpp:533-585) in one launch.  With stride_c == 0 and beta == 1 the
 * batch accumulates into one C (the broadcast-operand gradient); that case is
 * serialised internally so the sum is deterministic. */
int lten_hip_sgemm_strided_batched(int trans_a, int trans_b, uint64_t M, uint64_t N, uint64_t K, float alpha,
                                   const float* A, uint64_t lda, int64_t stride_a,
                                   const float* B, uint64_t ldb, int64_t stride_b, float beta,
                                   float* C, uint64_t ldc, int64_t stride_c, uint64_t batch);

/* FullyConnected forward in one launch: Y[M x out] = X[M x in] * W[out x in]^T (+ bias[out]),
 * i.e. the two cublasSgemm calls of l-ten/fully_connected.cpp:150,165 with the bias
 * rank-1 update folded into the epilogue.  bias may be NULL. */
int lten_hip_fc_forward_f32(uint64_t M, uint64_t in_features, uint64_t out_features, const float* X,
                            const float* W, const float* bias, float* Y);
/* The three GEMMs of fc_backward (l-ten/backprop.cpp:2228,2252,2267).  Any output may be
 * NULL.  dX and dW are overwritten (beta = 0); db accumulates (beta = 1), as in l-ten. */
int lten_hip_fc_backward_f32(uint64_t M, uint64_t in_features, uint64_t out_features, const float* X,
                             const float* W, const float* dY, float* dX, float* dW, float* db);

/* The same two calls with the relu that l-ten places around a hidden layer folded into the GEMM's store, so that a
 * training step needs fewer dependent launches (each costs about 5 us on this part whatever it computes):
 * lten_hip_fc_forward_relu_f32 writes the layer's output Y and Y_relu = relu(Y) (lten::relu of the result,
 * l-ten/layers.cpp:9-67; gpu_relu); lten_hip_fc_backward_relu_f32 applies relu_backward to the data gradient on the
 * way out, dX = relu_input > 0 ? (dY W) : 0 with relu_input[M x in] the input of the relu that produced X
 * (l-ten/backprop.cpp:2282-2327; gpu_relu_backward).  Same values as the unfused sequences, bit for bit. */
int lten_hip_fc_forward_relu_f32(uint64_t M, uint64_t in_features, uint64_t out_features, const float* X,
                                 const float* W, const float* bias, float* Y, float* Y_relu);
int lten_hip_fc_backward_relu_f32(uint64_t M, uint64_t in_features, uint64_t out_features, const float* X,
                                  const float* W, const float* dY, const float* relu_input, float* dX, float* dW,
                                  float* db);

/* ------------------------------------------------------------------ quantized GEMM */

/* GPU counterpart of quantized_matmul (l-ten/math_fns.h:104, l-ten/math_fns.cpp:1311-1478),
 * same argument list: C_u8[M x N] from A_u8, B_u8 (all four transpose modes), qparams[3] =
 * {A, B, C} (host memory), optional int32 bias[N] (device), int32 workspace[M + N]
 * (device scratch for the zero-point row/column terms; contents unspecified on return).
 * Operands outside the layout FullyConnected_q uses (transpose_a = 0, transpose_b = 1: both contiguous in K) or
 * with a K that is no multiple of 16 are first copied into that layout, rows padded, in memory the library owns
 * (allocated by the first such call, grown by later ones; not while a launch graph is being recorded, where such
 * calls run on a slower general kernel).
 * alpha != 1 or beta != 0 fail, as in l-ten (:1331-1334).  Outputs are bit-exact with the
 * CPU function wherever that function does not overflow int32 (K * 255^2 < 2^31) and
 * |real_multiplier * acc + zero_point| stays representable as a float. */
int lten_hip_quantized_matmul(int transpose_a, int transpose_b, uint64_t M, uint64_t N, uint64_t K,
                              uint8_t alpha, const uint8_t* A, const uint8_t* B, uint8_t beta, uint8_t* C,
                              const lten_hip_qparams* qparams, const int32_t* bias, int32_t* workspace);
/* Same computation, stopping before the requantize: acc[M x N] receives the corrected
 * int32 `element` of l-ten/math_fns.cpp:1469-1473.  For parity checks. */
int lten_hip_quantized_matmul_acc(int transpose_a, int transpose_b, uint64_t M, uint64_t N, uint64_t K,
                                  const uint8_t* A, const uint8_t* B, int32_t* acc,
                                  const lten_hip_qparams* qparams, const int32_t* bias, int32_t* workspace);
/* FullyConnected_q::forward's loop over leading dims (l-ten/fully_connected.cpp:373-396) as
 * one call: `batch` independent [M x in] inputs against one W[out x in]. workspace holds
 * batch * M + out ints. */
int lten_hip_fcq_forward(uint64_t batch, uint64_t M, uint64_t in_features, uint64_t out_features,
                         const uint8_t* X, const uint8_t* W, const int32_t* bias,
                         const lten_hip_qparams* qparams_in_wt_out, uint8_t* Y, int32_t* workspace);

/* Weights of a FullyConnected_q layer never change between forward calls (l-ten keeps them in the layer,
 * l-ten/fully_connected.cpp:301-303, and fills them once from a checkpoint).  lten_hip_fcq_prepare_weights, to be
 * called once when the layer moves to the GPU, turns the layer's uint8 weight bytes W[out_features][in_features]
 * into the int8 values w - 128 the matrix cores multiply, with every row on a 16-byte boundary: W_prepared holds
 * out_features rows of (in_features + 15) / 16 * 16 bytes, the bytes past in_features zero (both buffers 16-byte
 * aligned; in place when W_prepared == W and in_features is a multiple of 16, else the buffers may not overlap)
 * and, when weight_sums is not NULL, leaves each weight row's byte sum in weight_sums[out_features] (16-byte
 * aligned): the sums of the zero-point correction that quantized_matmul recomputes on every call
 * (l-ten/math_fns.cpp:1362-1369).  lten_hip_fcq_forward_prepared is lten_hip_fcq_forward on such weights and
 * returns bit-identical outputs.  For every shape the direct-to-LDS tiles take (in_features % 16 == 0 and >= 128,
 * more than 32 rows) it is a single launch whatever the zero points and the bias: the
 * column term comes from weight_sums, the activation rows' byte sums (needed when the weight zero point is not 128)
 * are added up from the operand fragments inside the GEMM.  When in_features is no multiple of 16 the activations
 * are first copied into rows of that length in memory the library owns (one more launch; the memory is allocated by
 * the first such call and grows with later ones, which cannot happen while a launch graph is being recorded), and
 * lten_hip_fcq_forward and lten_hip_quantized_matmul(0, 1, ...) copy both operands that way on every call.
 * The same memory holds the int32 sums of the chunks of K that at most 16 rows against an in_features above 16384
 * are computed in (one launch for the chunks, one that adds them; the tiled kernels take the call when the memory
 * cannot be had).
 * qparams are the layer's unchanged (the weight zero
 * point still refers to the uint8 representation).  workspace as for lten_hip_fcq_forward; only shapes that fall to
 * the general kernels use it.  No counterpart in l-ten, whose quantized layers are CPU-only. */
int lten_hip_fcq_prepare_weights(const uint8_t* W, uint8_t* W_prepared, uint64_t out_features, uint64_t in_features,
                                 int32_t* weight_sums);
int lten_hip_fcq_forward_prepared(uint64_t batch, uint64_t M, uint64_t in_features, uint64_t out_features,
                                  const uint8_t* X, const uint8_t* W_prepared, const int32_t* weight_sums,
                                  const int32_t* bias, const lten_hip_qparams* qparams_in_wt_out, uint8_t* Y,
                                  int32_t* workspace);

/* lten_hip_fcq_forward for callers that cannot allocate device memory or hand over a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in l-ten.  It calls no
 * hipMalloc / hipFree: the zero-point terms and, for small outputs with a long reduction, the split-K partial sums
 * and arrival counters live in one static device array of the library (8.3 MB per GPU, held until the process ends).
 * Limit: batch * M + out_features <= 65536; beyond it the call fails with a message.  Products whose partial sums
 * would not fit the array's 8 MB run unsplit.  Same outputs as lten_hip_fcq_forward, bit for bit.  Every call on a GPU
 * uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not. */
int lten_hip_fcq_forward_static(uint64_t batch, uint64_t M, uint64_t in_features, uint64_t out_features,
                                const uint8_t* X, const uint8_t* W, const int32_t* bias,
                                const lten_hip_qparams* qparams_in_wt_out, uint8_t* Y);

/* ------------------------------------------------------------------ im2col / conv */

/* Replace im2col_gpu<T> / col2im_gpu<T> (l-ten/im_col.h:60-73, l-ten/im_col.cu:98-118,164-184) in the three
 * instantiations l-ten compiles, float, int and uint8_t (l-ten/im_col.cu:199-218).  col is [C*kh*kw, Hout*Wout];
 * col2im overwrites im with the gathered sums, as the CUDA kernel does (l-ten/im_col.cu:123-162); integer sums
 * wrap as the template's `+=` on T does. */
int lten_hip_im2col_f32(const float* im, int channels, int height, int width, int kernel_h, int kernel_w,
                        int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                        float* col);
int lten_hip_im2col_i32(const int32_t* im, int channels, int height, int width, int kernel_h, int kernel_w,
                        int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                        int32_t* col);
int lten_hip_im2col_u8(const uint8_t* im, int channels, int height, int width, int kernel_h, int kernel_w,
                       int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                       uint8_t* col);
int lten_hip_col2im_f32(const float* col, int channels, int height, int width, int kernel_h, int kernel_w,
                        int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                        float* im);
int lten_hip_col2im_i32(const int32_t* col, int channels, int height, int width, int kernel_h, int kernel_w,
                        int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                        int32_t* im);
int lten_hip_col2im_u8(const uint8_t* col, int channels, int height, int width, int kernel_h, int kernel_w,
                       int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                       uint8_t* im);

/* Conv2d::forward's per-image im2col + cublasSgemm loop (l-ten/conv2d.cpp:164-171) as one
 * implicit-GEMM launch over the whole batch; no col buffer is materialised, except for layers
 * of many channels on small images (32 or more output channels, Cin*kh*kw >= 256, 32 or more
 * output pixels, no patch kernel for the shape, a cost estimate in favour), which follow l-ten's scheme
 * with the batch's column matrices (at most 512 MB) in memory the library owns: one im2col
 * launch, one strided batch of GEMMs, one pass for the bias.  Inside a graph recording that
 * route needs the memory to exist already (run the call once before recording it); otherwise
 * the implicit GEMM runs.
 * x[N,Cin,H,W], w[Cout,Cin*kh*kw], y[N,Cout,Hout,Wout]; bias[Cout] may be NULL
 * (l-ten adds it afterwards as a broadcast tensor add, l-ten/conv2d.cpp:189-192). */
int lten_hip_conv2d_forward_f32(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                                int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w,
                                const float* x, const float* w, const float* bias, float* y);
/* conv2_backward's weight branch (l-ten/backprop.cpp:1941-1954, the CPU semantics: the sum
 * over all images; the CUDA branch at :1989-2005 keeps only the last image and is not
 * followed).  dw[Cout, Cin*kh*kw] is overwritten.  workspace: device scratch of at least
 * lten_hip_conv2d_wgrad_workspace_bytes(...) bytes.  With at most 8192 output pixels in the
 * whole batch and many channels the gradient may instead be computed as one GEMM on copies of
 * the columns and of dy in memory the library owns (as for the forward pass). */
int lten_hip_conv2d_wgrad_f32(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                              int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w,
                              const float* x, const float* dy, float* dw, void* workspace);
uint64_t lten_hip_conv2d_wgrad_workspace_bytes(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                                               int kernel_h, int kernel_w, int pad_h, int pad_w,
                                               int stride_h, int stride_w);
/* conv2_backward's data branch (l-ten/backprop.cpp:1955-1968 CPU, :2007-2028 CUDA: per image col = W^T dy_n, then
 * col2im) for the whole batch: dx[N,Cin,H,W] is overwritten.  With stride 1 it runs as a convolution of dy with
 * the flipped, channel-transposed weights on the forward kernels; other strides run as one implicit GEMM over the
 * stride classes of the input pixels or, from a megabyte of columns on, as l-ten's GEMM + col2im done once for the
 * batch with the columns (at most 512 MB) in memory the library owns (inside a graph recording only if that memory
 * exists already: run the call once before recording it).  workspace: lten_hip_conv2d_dgrad_workspace_bytes(...)
 * device bytes. */
int lten_hip_conv2d_dgrad_f32(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                              int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w,
                              const float* w, const float* dy, float* dx, void* workspace);
uint64_t lten_hip_conv2d_dgrad_workspace_bytes(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                                               int kernel_h, int kernel_w, int pad_h, int pad_w,
                                               int stride_h, int stride_w);

/* Conv2d_q::forward (l-ten/conv2d.cpp:265-387; CPU-only in l-ten, "Conv2d_q only supports the CPU device
 * type" :376) for the whole batch: x[N][Cin][H][W] u8, w[Cout][Cin*kh*kw] u8, y[N][Cout][Ho][Wo] u8, with
 * qparams in the order input, weights, output (the layer's qparams_in_, qparams_wt_, qparams_out_; l-ten hands
 * them to quantized_matmul as [weights, input, output], :347-349).  Positions outside the image count as the
 * byte 0, as in l-ten's column buffer.  bias, when not null, holds Ho*Wo ints and is added per output position:
 * that is what l-ten's call computes (quantized_matmul indexes the bias by GEMM column, l-ten/math_fns.cpp:1470-1473,
 * and the columns of this product are output positions).  workspace: lten_hip_conv2dq_workspace_bytes device
 * bytes, 16-byte aligned.  Windows of at most 64 taps, and longer windows whose weights (of 32 output channels at
 * least) and a few input rows fit 64 KB of LDS, run in one launch and leave it untouched.  Other windows use it: the
 * patches of all output positions of the batch as rows
 * of a matrix, the padded weights, the int32 sums of one int8 GEMM over the whole batch and its zero-point terms;
 * where that would exceed 2 GiB, the column buffer of one image (l-ten's decomposition, image by image). */
uint64_t lten_hip_conv2dq_workspace_bytes(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout,
                                          int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w);
int lten_hip_conv2dq_forward(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kernel_h,
                             int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w, const uint8_t* x,
                             const uint8_t* w, const int32_t* bias, const lten_hip_qparams* qparams_in_wt_out,
                             uint8_t* y, void* workspace);
/* Same computation, stopping before the requantize (int32 `element` values).  For parity checks. */
int lten_hip_conv2dq_forward_acc(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kernel_h,
                                 int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w, const uint8_t* x,
                                 const uint8_t* w, const int32_t* bias, const lten_hip_qparams* qparams_in_wt_out,
                                 int32_t* acc, void* workspace);

/* ------------------------------------------------- element-wise pieces of a training step */

/* gpu_relu / gpu_relu_backward (l-ten/math_fns.h:231-234; l-ten/layers.cpp:9-67, l-ten/backprop.cpp:2282-2327):
 * dst = src > 0 ? src : 0;  bottom = input > 0 ? top : 0 (input = the relu's input). */
int lten_hip_relu_f32(float* dst, const float* src, uint64_t len);
int lten_hip_relu_backward_f32(float* bottom, const float* top, const float* input, uint64_t len);
/* gpu_mul(N, alpha, A, B) (l-ten/math_fns.h:137): y = alpha * x; what nll_backward is made of
 * (l-ten/backprop.cpp:3975-4040: bottom = (-1 / batch * top) * target). */
int lten_hip_scale_f32(uint64_t n, float alpha, const float* x, float* y);
/* cublasSaxpy as l-ten uses it to accumulate a leaf's gradient (l-ten/backprop.cpp:246-274): y += alpha * x. */
int lten_hip_axpy_f32(uint64_t n, float alpha, const float* x, float* y);
/* lten::log_softmax along the last dimension (l-ten/layers.cpp:93-114: max, sub, exp, sum, div, log as one kernel)
 * for x[rows][cols], and the sum of l-ten's backward functions of that chain: dx = dy - exp(y) * sum_j dy_j. */
int lten_hip_log_softmax_f32(uint64_t rows, uint64_t cols, const float* x, float* y);
int lten_hip_log_softmax_backward_f32(uint64_t rows, uint64_t cols, const float* y, const float* dy, float* dx);
/* gpu_nll (l-ten/math_fns.h:170; l-ten/layers.cpp:212-273): *loss = (sum_i input[i] * target[i]) * (-1 / batches). */
int lten_hip_nll_loss_f32(const float* input, const float* target, float* loss, uint64_t len, uint64_t batches);

/* Fewer launches around the loss, same values bit for bit: lten_hip_log_softmax_nll_loss_f32 = lten_hip_log_softmax_f32
 * followed by lten_hip_nll_loss_f32 (batches = rows); lten_hip_nll_log_softmax_backward_f32 = lten_hip_scale_f32(alpha,
 * target) followed by lten_hip_log_softmax_backward_f32, i.e. dx = alpha * target - exp(y) * sum_j alpha * target_j with
 * alpha = -top / rows for l-ten's nll_backward (l-ten/backprop.cpp:3975-4040); lten_hip_log_softmax_nll_loss_grad_f32 =
 * both of them.  The first and the third are one launch for up to 1024 rows of up to 16 columns (a classifier's
 * logits) and the separate launches otherwise. */
int lten_hip_log_softmax_nll_loss_f32(uint64_t rows, uint64_t cols, const float* x, const float* target, float* y, float* loss);
int lten_hip_nll_log_softmax_backward_f32(uint64_t rows, uint64_t cols, const float* y, const float* target, float alpha, float* dx);
int lten_hip_log_softmax_nll_loss_grad_f32(uint64_t rows, uint64_t cols, const float* x, const float* target, float alpha, float* y,
                                           float* loss, float* dx);

/* The loss and the backward pass of the layer that produced the logits, in one launch: lten_hip_log_softmax_nll_loss_grad_f32
 * (rows = M, cols = out_features, x = logits; writes log_probs, *loss and dlogits) followed by lten_hip_fc_backward_f32 with
 * dY = dlogits (l-ten/layers.cpp:93-114,212-273; l-ten/backprop.cpp:3975-4040,2083-2280), or, with relu_input not NULL,
 * by lten_hip_fc_backward_relu_f32; same values bit for bit.  One launch for a classifier's last layer (out_features <= 16,
 * M * out_features <= 4096, M < 512, dX and dW both wanted), the separate launches otherwise. */
int lten_hip_fc_backward_log_softmax_nll_loss_f32(uint64_t M, uint64_t in_features, uint64_t out_features, const float* X, const float* W,
                                                  const float* logits, const float* target, float alpha, float* log_probs, float* loss,
                                                  float* dlogits, const float* relu_input, float* dX, float* dW, float* db);

/* gpu_sgd_step (l-ten/math_fns.h:186; SGDOptimizer::step, l-ten/optimizer.cpp:26-84) for one parameter tensor:
 * grad = wd * w + grad (stored, as in l-ten), velocity = velocity * mo + (1 - mo) * grad, w = w - velocity * lr. */
int lten_hip_sgd_step_f32(float* weight, float* weight_grad, float* velocity, uint64_t numels, float mo, float wd, float lr);
/* AdamOptimizer::step (l-ten/optimizer.cpp:107-186) for one parameter tensor: l-ten's eight element-wise launches
 * (gpu_axpby, gpu_mul, gpu_axpby, gpu_mul, gpu_powx, gpu_add, gpu_div, gpu_axpy) as one pass.  v_dw and s_dw are the
 * first two thirds of l-ten's history tensor; its last third (scratch) is not needed.  iteration counts from 1. */
int lten_hip_adam_step_f32(float* weight, const float* weight_grad, float* v_dw, float* s_dw, uint64_t numels, float lr,
                           float beta1, float beta2, uint64_t iteration);

/* The gradient of a Conv2d bias: db[c] = (accumulate ? db[c] : 0) + sum over n, h, w of dy[n][c][h*w].  l-ten adds the
 * bias {1, C, 1, 1} to the convolution's result as a tensor op (l-ten/conv2d.cpp:189-192), so this is the backward
 * pass of that broadcast add (l-ten/backprop.cpp:605-690: the top gradient summed over the broadcast dimensions).
 * Up to 4096 channels; two launches, partial sums in a device array of the library. */
int lten_hip_conv2d_bias_grad_f32(uint64_t N, uint64_t C, uint64_t HW, const float* dy, float* db, int accumulate);

/* ------------------------------------------------------------------ quantization helpers */

/* Quantize / Dequantize / GetMinMax of l-ten/utils.h:23-26 (l-ten/utils.cpp:198-262) with the data on the device;
 * bit-exact with the CPU functions.  qparams is a host pointer.  lten_hip_get_min_max returns its two results to
 * host memory and synchronises; ComputeQuantizationParams (two floats in, one QuantizationParams out) stays host code. */
int lten_hip_quantize_u8(const float* data, uint8_t* q_data, uint64_t len, const lten_hip_qparams* qparams);
int lten_hip_quantize_i32(const float* data, int32_t* q_data, uint64_t len, const lten_hip_qparams* qparams);
int lten_hip_dequantize_u8(float* data, const uint8_t* q_data, uint64_t len, const lten_hip_qparams* qparams);
int lten_hip_get_min_max(const float* data, uint64_t len, float* min_val, float* max_val);

/* ----------------------------------------------------------------------- launch graphs */

/* A training or inference step is a fixed sequence of short launches (twenty for a three-layer MLP step), and
 * the host's launch cost then exceeds the kernels' run time.  lten_hip_graph_begin starts recording the
 * compute entry points called on this thread instead of running them; lten_hip_graph_end returns the
 * recording as a handle, and every lten_hip_graph_launch replays it on the library's stream with one submit.
 * Pointers and sizes are recorded by value: the buffers must stay where they are (new contents are fine).
 * Between begin and end only compute entry points may be called: lten_hip_alloc / free / copy_* / sync /
 * set_stream / get_min_max / event_elapsed_ms fail with a message (they allocate, copy or wait, which a recording
 * cannot hold), and lten_hip_last_kernel names
 * what was recorded, not what ran.  When the library is on the null stream the recording uses a stream of
 * the library's own; replays still go to the library's stream.  One capture at a time per process.  A buffer a
 * recording names must not be handed to lten_hip_free while the handle lives (the pool would give it to the next
 * lten_hip_alloc); lten_hip_graph_destroy waits for the stream before it lets go of the recording.
 * No counterpart in l-ten, whose GPU branches launch eagerly on the default stream. */
int lten_hip_graph_begin(void);
int lten_hip_graph_end(void** graph);
int lten_hip_graph_launch(void* graph);
int lten_hip_graph_destroy(void* graph);

/* ----------------------------------------------------------------------- measurement */

/* HIP events on the library's stream; no counterpart in l-ten (its benchmarks use
 * steady_clock around synchronous calls). */
int lten_hip_event_create(void** event);
int lten_hip_event_record(void* event);
int lten_hip_event_elapsed_ms(void* start, void* stop, float* ms); /* synchronises on `stop` */
int lten_hip_event_destroy(void* event);

/* Kernel-selection override for tests and tuning sweeps; 0 restores the built-in heuristic.
 * Options: "qgemm_tile", "sgemm_tile", "qskinny", "conv_variant", "qgemm_split".  No counterpart in l-ten. */
int lten_hip_set_option(const char* name, int value);

/* Name of the kernel variant the last GEMM-type call on this thread dispatched to
 * (e.g. "qgemm_nt_256x256x64"); for reports and tests. */
const char* lten_hip_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* LTEN_HIP_H */
