/*
 * nz_oracle.h -- CPU restatement of NeuZephyr's tensor-core GEMM path.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker for the HIP library and the
 * timed CPU baseline of the benchmark; nothing in the shipped library links,
 * loads or calls it.
 *
 * Every function cites the reference file:line it restates (paths are relative
 * to the NeuZephyr source tree).  The reference itself is CUDA-only (nvcc,
 * <mma.h>, cuRAND) and cannot be compiled here, so each function is pinned by
 * the reference's own literal test vectors, by hardware F16C conversion, and
 * by closed forms / brute force (see tests/test_oracle_*.py).
 *
 * Parity status:
 *   - fp32->fp16 rounding ............ pinned (F16C hardware, exhaustive halfs)
 *   - GEMM / batched broadcast GEMM .. pinned (reference literal vectors,
 *                                      integer exactness, fp64 truth bound)
 *   - im2col / col2im ................ pinned (reference loop-nest spec,
 *                                      direct-convolution identity)
 *   - bias add / ReLU ................ pinned (closed form, NaN / -0 cases)
 *   - backward (GEMM, add, ReLU, im2col, col2im) pinned (reference literal vectors
 *                                      Test.cpp:820-903, loop nests :3011-3072 and
 *                                      :3144-3177, adjoint identities <Jv,u> = <v,J^T u>)
 *   - fp32 matmul, SGD ............... pinned (reference literal vector Test.cpp:119-184, closed form);
 *                                      whether each k step is one FMA or a rounded multiply and add is
 *                                      the CUDA compiler's choice (default: FMA, restated here): the last
 *                                      bit of non-integer results is PARITY UNPINNED
 *   - Adam ........................... pinned against the host formula of the reference's own test
 *                                      (Test.cpp:2398-2452); the kernel's __powf bits: PARITY UNPINNED
 *   - bit-level accumulation order of nvcuda::wmma::mma_sync: PARITY UNPINNED
 *     (unspecified by the vendor; the tolerance contract replaces it).
 */
#ifndef NZ_ORACLE_H
#define NZ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 rounding: __float2half in Padding, src/OperationKernels.cu:846-860 */
uint16_t nzo_f32_to_f16_bits(float x);          /* IEEE RNE, subnormals kept, >=65520 -> inf */
float nzo_f16_bits_to_f32(uint16_t h);
float nzo_round_f16(float x);                   /* f16_bits_to_f32(f32_to_f16_bits(x)) */
void nzo_round_f16_array(float* dst, const float* src, size_t n);

/* ---- single GEMM: GeneralMatrixMulTensorKernel, src/OperationKernels.cu:821-844
 * C[M,N] = f16(A)[M,K] * f16(B)[K,N], fp32 accumulation, k ascending.
 * trans_b != 0: B is given as N x K row-major (element (k,n) at B[n*ldb+k]).
 * Zero padding to multiples of 16 (utils.cuh:13) adds exact zeros and is
 * therefore not materialised. */
void nzo_gemm_f16in_f32acc(const float* A, const float* B, float* C,
                           size_t M, size_t N, size_t K,
                           size_t lda, size_t ldb, size_t ldc, int trans_b);

/* Same rounded inputs, fp64 accumulation: the truth the tolerances refer to. */
void nzo_gemm_f16in_f64acc(const float* A, const float* B, double* C,
                           size_t M, size_t N, size_t K,
                           size_t lda, size_t ldb, size_t ldc, int trans_b);

/* Rows [row0,row0+nrows) only, fp32 and fp64 accumulation (sampling of big cases). */
void nzo_gemm_rows(const float* A, const float* B, float* C32, double* C64,
                   size_t row0, size_t nrows, size_t N, size_t K,
                   size_t lda, size_t ldb, int trans_b);

/* ---- batched driver: TensorCoreGEMMParallel, src/OperationKernels.cu:914-1026
 * shapes are {n,c,h,w}; M=A.h, N=B.w, K=A.w; loops over C's (n,c); an operand
 * whose n (or c) is 1 is broadcast along that axis (:981-984). */
void nzo_tensorcore_gemm(const float* A, const float* B, float* C,
                         const size_t shapeA[4], const size_t shapeB[4], const size_t shapeC[4]);

/* fp32-exact matmul behind Tensor::operator*: GeneralMatrixMulKernel,
 * src/OperationKernels.cu:65-101 (comparator only; no fp16 rounding). */
void nzo_general_matmul(const float* A, const float* B, float* C,
                        const size_t shapeA[4], const size_t shapeB[4], const size_t shapeC[4]);

/* ---- im2col: img2colKernel, src/OperationKernels.cu:1308-1328 */
void nzo_im2col(float* out, const float* in, size_t H_out, size_t W_out, size_t C,
                size_t K_h, size_t K_w, size_t stride, size_t pad,
                size_t H_in, size_t W_in, size_t batch);

/* ---- col2im: col2imgKernel, src/OperationKernels.cu:1364-1376 */
void nzo_col2im(float* out, const float* in, size_t H_out, size_t W_out, size_t C_out, size_t batches);

/* ---- broadcast add: tensorMatrixAdd + MatrixAddKernel,
 * include/NeuZephyr/TensorOperations.cuh:785-808, src/OperationKernels.cu:12-24 */
void nzo_matrix_add(float* out, const float* a, const float* b,
                    const size_t shapeOut[4], const size_t shapeA[4], const size_t shapeB[4]);

/* ---- ReLU: RectifiedLinearUnitKernel, src/OperationKernels.cu:230-235 (x>0?x:0) */
void nzo_relu(float* out, const float* in, size_t n);

/* ---- Model::Conv2d graph, src/Model.cu:244-263 (+ optional trailing ReLU node):
 * x[N,C,H,W]; w_ref[Wb,1,C*Kh*Kw,O] with Wb in {1,N}; bias_ref[1,1,Ho*Wo,O] or NULL;
 * y[N,O,Ho,Wo].  Runs im2col -> GEMM -> add -> col2im (-> ReLU) exactly as the
 * reference graph does, materialising the intermediates. */
void nzo_conv2d_graph(float* y, const float* x, const float* w_ref, const float* bias_ref,
                      size_t N, size_t C, size_t H, size_t W, size_t O,
                      size_t K_h, size_t K_w, size_t stride, size_t pad,
                      size_t w_batch, int relu);

/* Independent 7-loop direct convolution of the fp16-rounded operands in fp64,
 * OIHW weights, per-channel bias (NULL ok).  Used to pin nzo_conv2d_graph. */
void nzo_conv2d_direct_f64(double* y, const float* x, const float* w_oihw, const float* bias_o,
                           size_t N, size_t C, size_t H, size_t W, size_t O,
                           size_t K_h, size_t K_w, size_t stride, size_t pad, int relu);

/* ---- Model::Linear graph, src/Model.cu:87-103 (+ optional ReLU):
 * y[n][o] = relu(sum_i f16(Wt[o][i]) * f16(x[n][i]) + bias[o]); Wt is [OUT,IN]. */
void nzo_linear_graph(float* y, const float* x, const float* w_out_in, const float* bias,
                      size_t batch, size_t in_features, size_t out_features, int relu);

/* ---- error metrics used by the tolerance contract */
/* ---- backward of the same path -------------------------------------------
 * GEMMBackwardParallel, src/OperationKernels.cu:1028-1144 (+ CuttingAndCompress :873-883):
 * for every (i,j) of the batch max(A,B):  C[i or 0][j or 0] += f16(A_ij)[M,K] * f16(B_ij)[K,N]
 * (fp32 accumulation per product, k ascending; products ADDED to what C holds, members of a
 * reduced batch dimension in ascending order -- the reference's atomicAdd leaves that order open). */
void nzo_gemm_backward(const float* A, const float* B, float* C, const size_t shapeA[4],
                       const size_t shapeB[4], const size_t shapeC[4]);
/* MatMulNode::backward, src/Nodes.cu:169-182: dA += dC * B^T, dB += A^T * dC through explicit
 * transposes (TransposeKernel, OperationKernels.cu:125-145) and nzo_gemm_backward.  dA / dB may be NULL. */
void nzo_matmul_backward(float* dA, float* dB, const float* A, const float* B, const float* dC,
                         const size_t shapeA[4], const size_t shapeB[4], const size_t shapeC[4]);
/* ReLUBackwardKernel, src/OperationKernels.cu:242-248: dx = x > 0 ? dy : 0 (overwrites). */
void nzo_relu_backward(float* dx, const float* x, const float* dy, size_t n);
/* AddNode::backward for one input, src/Nodes.cu:99-146: equal shapes -> copy (overwrite);
 * otherwise din[n or 0][c or 0][:] += dout[n][c][:] for every (n,c) (gradCopyKernel :1230-1236). */
void nzo_add_backward(float* din, const float* dout, const size_t shapeIn[4], const size_t shapeOut[4]);
/* img2colBackwardKernel, src/OperationKernels.cu:1337-1355: every column-matrix gradient element is
 * ADDED to the image gradient element it was copied from (padding positions dropped). */
void nzo_im2col_backward(float* dx, const float* dcol, size_t H_out, size_t W_out, size_t C, size_t K_h,
                         size_t K_w, size_t stride, size_t pad, size_t H_in, size_t W_in, size_t batch);
/* col2imgBackwardKernel, src/OperationKernels.cu:1384-1396: dcol[b][(h*W+w)*C+c] = dy[b][c][h][w]. */
void nzo_col2im_backward(float* dcol, const float* dy, size_t H_out, size_t W_out, size_t C_out, size_t batches);
/* dx += data gradient of the stride-1 Conv2d graph (the chain Nodes.cu:660-665 -> :169-182 -> :632-640 in one
 * statement); dy [N,O,H_out,W_out], w_ref [w_batch,1,C*K_h*K_w,O], dx [N,C,H,W]. */
/* dw += weight gradient of the stride-1 Conv2d graph (Nodes.cu:169-182 on the column matrix of :605-630);
 * x [N,C,H,W], dy [N,O,H_out,W_out], dw [w_batch,1,C*K_h*K_w,O]. */
void nzo_conv2d_backward_weights_strided(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H,
                                         size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                         size_t w_batch);
void nzo_conv2d_backward_weights(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H, size_t W,
                                 size_t O, size_t K_h, size_t K_w, size_t pad, size_t w_batch);
/* dx += data gradient of the Conv2d graph (Nodes.cu:660-665, 169-182, 632-640); dy [N,O,H_out,W_out], dx [N,C,H,W]. */
void nzo_conv2d_backward_data_strided(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H,
                                      size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                      size_t w_batch);
void nzo_conv2d_backward_data(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H,
                              size_t W, size_t O, size_t K_h, size_t K_w, size_t pad, size_t w_batch);

/* ---- softmax -------------------------------------------------------------
 * Host statement of the reference's own tests (test/Test.cpp:1823-1832, 1782-1795): exp / sum(exp)
 * per contiguous vector with the sum taken in ascending order, and the Jacobian loop nest. The kernels
 * use __expf and a tree sum: their last bits are PARITY UNPINNED (the tests compare at 1e-5). */
void nzo_softmax(float* out, const float* in, size_t len, size_t batch);
void nzo_softmax_jacobian(float* out, const float* in, size_t n, size_t batch);

/* ---- optimizer steps ------------------------------------------------------
 * StochasticGradientDescentKernel, src/OperationKernels.cu:634-640: data -= lr * grad. */
void nzo_sgd_step(float* data, const float* grad, float lr, size_t n);
/* AdamKernel, src/OperationKernels.cu:753-766 (fp32 throughout). beta^t through powf: the reference
 * uses CUDA's approximate __powf there, whose last bits are PARITY UNPINNED. */
void nzo_adam_step(float* data, float* m, float* v, const float* grad, float lr, float beta1, float beta2,
                   float eps, int t, size_t n);

/* ---- average pooling, binary cross-entropy, expand / compress -----------------
 * AveragePoolingKernel (src/OperationKernels.cu:1404-1429), which is also the loop nest of the reference's
 * own test (test/Test.cpp:3179-3246): mean over the window cells inside the image, row by row. */
void nzo_avgpool2d(float* out, const float* in, size_t pool, size_t stride, size_t pad, size_t batches,
                   size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out);
/* AveragePoolingBackwardKernel (:1439-1486) run serially in ascending output index: din += dout / divisor
 * (pool^2 without padding, the in-image cell count with padding). The reference's atomicAdd order is not
 * defined; a serial run is one of its possible orders. */
void nzo_avgpool2d_backward(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches,
                            size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out);
/* Mean binary cross-entropy as the reference's test states it (test/Test.cpp:1955-1958): the terms summed in
 * ascending order with logf, then divided by n. The kernel (:648-685) divides every term by n, uses __logf
 * and a tree sum: last bits are PARITY UNPINNED (the reference's test compares at 1e-2). */
float nzo_bce_loss(const float* predict, const float* real, size_t n);
/* BCEBackwardKernel (:692-699; test/Test.cpp:1985-1987): ((p - t) / (p (1 - p))) / n. */
void nzo_bce_backward(float* grad, const float* predict, const float* real, size_t n);
/* Mean squared error as the reference's test states it (test/Test.cpp:1890-1893): squared differences summed in
 * ascending order, then divided by n (the kernel, :579-619, divides every term and sums in a tree: last bits
 * PARITY UNPINNED, the test compares at 1e-2); MSEBackwardKernel (:621-627): 2 (p - t) / n. */
float nzo_mse_loss(const float* predict, const float* real, size_t n);
void nzo_mse_backward(float* grad, const float* predict, const float* real, size_t n);
/* ExpandKernel / CompressKernel (:1282-1301), the latter run serially in ascending index. */
void nzo_expand(float* out, const float* in, size_t n, size_t batches);
void nzo_compress(float* out, const float* in, size_t n, size_t batches);

/* max over i of |got-truth| / max(|truth|, floor) and Frobenius ||got-truth|| / ||truth|| */
void nzo_errors_f32_vs_f64(const float* got, const double* truth, size_t n, double floor_abs,
                           double* max_rel, double* frob_rel);

/* ---- seeded generators (documented PRNG: splitmix64-seeded xoshiro256**, one
 * independent stream per block of 4096 elements so generation parallelises;
 * normals by Box-Muller in double). kind: 0 uniform[lo,hi), 1 normal(mean=lo, std=hi) */
void nzo_fill(float* dst, size_t n, uint64_t seed, int kind, double lo, double hi);

int nzo_num_threads(void);
void nzo_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
