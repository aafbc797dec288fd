/*
 * nzhip.h -- C-ABI of the MI355X (gfx950) implementation of NeuZephyr's
 * tensor-core GEMM path: fp32 operands rounded to fp16 (round-to-nearest-even),
 * fp16 MFMA with fp32 accumulation, and what feeds and drains it (im2col,
 * col2im, bias add, ReLU, Conv2d lowering, device allocator, stream manager).
 *
 * Conventions
 *   - every pointer named A/B/C/in/out/x/w/y/bias is a DEVICE pointer (or pinned
 *     host memory mapped into the device) to contiguous fp32 data owned by the
 *     caller; the library never takes ownership;
 *   - `stream` is a hipStream_t passed as void*; NULL is HIP's null stream.  All
 *     compute entry points only enqueue work and return before it completes;
 *   - return value: 0 = ok, negative = NZHIP_E_* (invalid argument etc., nothing
 *     was enqueued), positive = a hipError_t raised by the runtime.  Nothing is
 *     thrown across this boundary.  nzhip_last_error() returns a thread-local,
 *     human-readable description of the last non-zero status;
 *   - shapes given as size_t[4] are NeuZephyr Dimensions {n, c, h, w} of
 *     contiguous NCHW tensors (reference: src/Dimension.cu:5-10).
 *
 * Line numbers cite the NeuZephyr sources each entry point replaces.
 */
#ifndef NZHIP_H
#define NZHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NZHIP_OK 0
#define NZHIP_E_INVALID (-1)      /* bad pointer / size / stride / enum */
#define NZHIP_E_SHAPE (-2)        /* shapes are not broadcast compatible */
#define NZHIP_E_UNSUPPORTED (-3)  /* valid request outside implemented limits */
#define NZHIP_E_NOMEM (-4)        /* device allocation failed */
#define NZHIP_E_TIMEOUT (-5)      /* an earlier single-kernel product ran out of polls; see nzhip_gemm_coop_timeouts */

#define NZHIP_ACT_NONE 0
#define NZHIP_ACT_RELU 1          /* x > 0 ? x : 0  (NaN -> 0, -0 -> +0) */

#define NZHIP_LAYOUT_ROW 0        /* operand as written: A is MxK, B is KxN, row-major */
#define NZHIP_LAYOUT_TRANS 1      /* operand given transposed: A as KxM, B as NxK, row-major */

/* ---- library ------------------------------------------------------------ */
int nzhip_version(void);
const char* nzhip_last_error(void);
/* Device properties the library keys its launch shapes on (CU count, LDS per CU);
 * 0 on success.  Also the cheapest "is a gfx950 GPU usable" probe. */
int nzhip_device_info(int* cu_count, size_t* lds_bytes_per_cu, char* arch_name, size_t arch_name_len);

/* ---- GEMM --------------------------------------------------------------- */
/* General form of the path's one contraction.  For every (i, j) of a two-level
 * batch (batch_n x batch_c):
 *     C_ij[M,N] = act( f16(A_ij)[M,K] * f16(B_ij)[K,N] + bias_ij )
 * with fp32 accumulation.  Replaces Padding + GeneralMatrixMulTensorKernel +
 * Cutting (src/OperationKernels.cu:821-871) and the per-(n,c) launch loops of
 * TensorCoreGEMMParallel (:914-1026); the fused bias/activation replaces
 * MatrixAddKernel (:12-24) and RectifiedLinearUnitKernel (:230-235).
 * Edges are predicated in-kernel: no padded copies exist.
 * Strides are in elements; a batch stride of 0 broadcasts that operand.
 * bias may be NULL; its element for output (m,n) of batch (i,j) is
 *     bias[i*bias_stride_n_batch + j*bias_stride_c_batch + m*bias_stride_row + n*bias_stride_col]
 * so a per-row vector, a per-column vector and a full [M,N] matrix are all expressible.
 * bias may be C itself with C's strides ("C += A*B", how the backward entry points accumulate): on every
 * route the thread that stores C(m,n) is the one that read bias(m,n) before.  Any other overlap of bias
 * and C, and any overlap of A or B with C, is undefined. */
typedef struct nzhip_gemm_desc {
    const float* A;
    const float* B;
    float* C;
    int64_t M, N, K;
    int64_t lda, ldb, ldc;        /* leading dimensions (row strides) of the arrays as stored */
    int32_t a_layout;             /* NZHIP_LAYOUT_ROW: A[m*lda+k];  _TRANS: A[k*lda+m] */
    int32_t b_layout;             /* NZHIP_LAYOUT_ROW: B[k*ldb+n];  _TRANS: B[n*ldb+k] */
    int64_t batch_n, batch_c;     /* >= 1 */
    int64_t a_stride_n, a_stride_c;
    int64_t b_stride_n, b_stride_c;
    int64_t c_stride_n, c_stride_c;
    const float* bias;            /* optional */
    int64_t bias_stride_row, bias_stride_col;
    int64_t bias_stride_n, bias_stride_c;
    int32_t activation;           /* NZHIP_ACT_* */
    int32_t reserved;             /* must be 0 */
} nzhip_gemm_desc;

int nzhip_gemm(const nzhip_gemm_desc* desc, void* stream);

/* nzhip_gemm for callers that cannot allocate device memory (tight serving loops, harnesses that
 * forbid hipMalloc, code that is to run under HIP graph capture -- not tested under capture here; the first
 * call on a device looks up the static array's address and raises kernels' dynamic-LDS limits, which are
 * driver calls, so make one call of each shape class outside a capture first).  No counterpart in the
 * reference, whose GEMM
 * driver allocates three temporaries per call (src/OperationKernels.cu:885-912).
 * Same arguments, same kernels and bit-identical results, but every workspace the routes use
 * (fp16 operand images of the two-pass route, split-contraction partial sums, padded copies of
 * operands whose rows do not allow 16-byte loads) lives in a static device array of
 * NZHIP_STATIC_SCRATCH_BYTES that each GPU holds from library load until the process ends; the
 * call performs no hipMalloc / hipFree and never touches the caching pool.
 * A product whose workspace would not fit is rejected with NZHIP_E_UNSUPPORTED
 * (nzhip_last_error() names the size) and leaves C untouched.  The one workspace that is only
 * an optimisation, the padded operand copies, is given up instead when it does not fit: the
 * product is then computed from the operands as given, and its sums may be grouped differently
 * from nzhip_gemm's (same tolerance, not the same last bits).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race; serialise them. */
#define NZHIP_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int nzhip_gemm_static(const nzhip_gemm_desc* desc, void* stream);
size_t nzhip_static_scratch_bytes(void);

/* Test and benchmark hook (no counterpart in the reference): nzhip_gemm with the kernel chosen by the
 * caller instead of by the shape, so that every kernel can be checked on every shape.
 * tile 64 / 128 / 256: the fused convert-on-load kernel with that square tile; 16 / 18 / 12: the two-pass
 * fp16 route with 256x256 tiles on 4 waves / 256x256 tiles on 8 waves / 128x256 tiles, 16x16x32 MFMAs;
 * 316 / 318 / 312: the same three with 32x32x16 MFMAs; 28: the single-kernel route for very large
 * products (rounding overlapped with the MFMA loop; NZHIP_E_UNSUPPORTED unless M and N are multiples of
 * 4096 and K of 1024).  Any other value: NZHIP_E_INVALID. */
int nzhip_gemm_force_tile(const nzhip_gemm_desc* desc, int tile, void* stream);
/* Diagnostic (no counterpart in the reference): in the single-kernel route workgroups wait for each
 * other's rounding work with a bounded number of polls; *count receives how many waits have run out
 * since the library was loaded (expected: 0; anything else means a device with fewer than 256 free
 * compute units, e.g. one shared with another process or stream).  Blocks until the device is idle.
 * What C holds after a wait ran out: every workgroup looks at the launch's own count of such waits in
 * front of its result stores, and from the first one on every 256 x 256 tile of C is written as NaN
 * (tiles stored before it are complete and correct).  A product of this route can therefore be wrong
 * only visibly, whichever stream it ran on and however the caller synchronises.
 * The runtime looks at the process-wide count by itself as well: the first nzhip_sync_ptr,
 * nzhip_sync_all or nzhip_memcpy_d2h that has drained the stream of such a product returns
 * NZHIP_E_TIMEOUT once if the count went up (the copy or wait itself has been carried out: after
 * nzhip_memcpy_d2h the destination is filled), and from then on nzhip_gemm keeps to the two-kernel
 * route in this process. */
int nzhip_gemm_coop_timeouts(unsigned* count);
/* Test hook for that report: adds `inject` to the device-side count as if that many waits had run out
 * (no kernel misbehaves), or, with inject == 0, forgets earlier time-outs (the count reads 0 again) and allows the route again. */
int nzhip_gemm_coop_reset(unsigned inject);
/* Test hook for the waits themselves: spin_limit polls per wait (0 = the default, a few hundred ms) and,
 * with mute != 0, workgroups that keep their arrivals to themselves, so that every wait of the following
 * single-kernel products runs out after spin_limit polls.  All waves still run to the end of the kernel;
 * the product comes out as NaN.  Always returns NZHIP_OK. */
int nzhip_gemm_coop_test_mode(unsigned spin_limit, int mute);

/* ---- prepared operands ---------------------------------------------------------------------------------
 * No counterpart in the reference, which rounds and pads both operands anew on every call
 * (src/OperationKernels.cu:940-975).  Several routes first turn an operand into an fp16 image: the two-pass
 * GEMM route its B operand, the implicit-GEMM convolution kernels their weights.  A layer's weights do not
 * change between forward calls, so a caller may keep that image in a handle: the first call through a handle
 * builds the image into memory the handle owns, later calls with the same operand (address, extents, layout,
 * and a route that wants the same image) skip the conversion kernel; anything else rebuilds it.  Routes
 * without an image (skinny, fused convert-on-load, single-kernel, direct and column-matrix convolutions)
 * ignore the handle.  Results are bit-identical with and without a handle.
 * The library cannot see writes to the operand: after the weights change, call nzhip_prepared_invalidate
 * before the next product (a stale image gives the product of the OLD weights, silently).
 * A handle's image is filled on the stream of the call that builds it; use a handle on one stream at a time
 * (or synchronise that stream before using the handle elsewhere).  nzhip_prepared_destroy returns the image
 * to the pool in the order of that stream.  nzhip_prepared_fills: how often an image has been built through
 * the handle (tests, tuning). */
typedef struct nzhip_prepared nzhip_prepared;
int nzhip_prepared_create(nzhip_prepared** handle);
int nzhip_prepared_invalidate(nzhip_prepared* handle);
int nzhip_prepared_fills(const nzhip_prepared* handle, unsigned long long* count);
int nzhip_prepared_destroy(nzhip_prepared* handle);
/* nzhip_gemm with the image of B kept in b_image (NULL: plain nzhip_gemm). */
int nzhip_gemm_prepared_b(const nzhip_gemm_desc* desc, nzhip_prepared* b_image, void* stream);

/* Measurement hooks (no counterpart in the reference; not used by any product path): what the GPU at hand
 * sustains with only its matrix pipes, or only its memory system, at work -- the two figures a benchmark
 * sets a kernel's rate against, next to the published peaks.
 * nzhip_probe_mfma: one workgroup of four waves per compute unit; every wave issues `passes` x 64
 * v_mfma_f32_16x16x32_f16 on fragments held in registers (a fixed pseudo-random fp16 pattern, or zeros with
 * zero_operands != 0), i.e. cu_count x 4 x passes x 64 x 16384 flop per call; time it with events on
 * `stream`.  `workspace`: device memory of NZHIP_PROBE_MFMA_WORKSPACE_BYTES, 16-byte aligned; after the call
 * its first 2 x cu_count 64-bit words hold, per workgroup, the elapsed shader-clock ticks and the elapsed ticks
 * of the constant 100 MHz counter of the loop (ticks ratio x 100 MHz = the clock the chip held under the loop).
 * nzhip_probe_copy: dst[0, bytes) = src[0, bytes) with 16-byte accesses (both 16-byte aligned, bytes a
 * multiple of 16): 2 x bytes of memory traffic per call. */
#define NZHIP_PROBE_MFMA_WORKSPACE_BYTES ((size_t)65536)
int nzhip_probe_mfma(int passes, int zero_operands, void* workspace, size_t workspace_bytes, void* stream);
int nzhip_probe_copy(void* dst, const void* src, size_t bytes, void* stream);

/* Drop-in for nz::data::iTensorCoreGEMM (include/NeuZephyr/TensorOperations.cuh:1021-1022,
 * src/TensorOperations.cu:112-115 -> krnl::TensorCoreGEMMParallel, src/OperationKernels.cu:914-1026):
 * M = A.h, N = B.w, K = A.w; loops over C's (n,c); an operand whose n (or c) is 1 is
 * broadcast.  Like the reference it validates nothing beyond non-null pointers. */
int nzhip_tensorcore_gemm(const float* A, const float* B, float* C, const size_t shapeA[4],
                          const size_t shapeB[4], const size_t shapeC[4], void* stream);

/* ---- conv lowering ------------------------------------------------------ */
/* nz::data::iImg2col (TensorOperations.cuh:1108-1110; img2colKernel, OperationKernels.cu:1308-1328):
 * out[b][ho*W_out+wo][c*K_h*K_w + r*K_w + s] = in[b][c][ho*stride-pad+r][wo*stride-pad+s] or 0. */
int nzhip_im2col(float* out, const float* in, size_t H_out, size_t W_out, size_t C, size_t K_h,
                 size_t K_w, size_t stride, size_t pad, size_t H_in, size_t W_in, size_t batch,
                 void* stream);

/* nz::data::iCol2img (TensorOperations.cuh:1132-1133; col2imgKernel, OperationKernels.cu:1364-1376):
 * out[b][c][h][w] = in[b][(h*W_out+w)*C_out + c]. */
int nzhip_col2im(float* out, const float* in, size_t H_out, size_t W_out, size_t C_out, size_t batches,
                 void* stream);

/* The whole Model::Conv2d graph (src/Model.cu:244-263: Img2Col -> MatMul -> Bias -> Col2Img,
 * optionally followed by the ReLU node) as one fused call with no column matrix in HBM.
 *   x      [N, C, H, W]
 *   w_ref  [w_batch, 1, C*K_h*K_w, O], w_batch in {1, N}; row q = c*K_h*K_w + r*K_w + s
 *   bias   optional; element for output (b, o, p = ho*W_out+wo) is
 *          bias[p*bias_stride_pixel + o*bias_stride_channel]
 *          (reference parameter [1,1,H_out*W_out,O]: pixel stride O, channel stride 1;
 *           ordinary per-channel vector: pixel stride 0, channel stride 1)
 *   y      [N, O, H_out, W_out] */
int nzhip_conv2d_forward(float* y, const float* x, const float* w_ref, const float* bias,
                         size_t N, size_t C, size_t H, size_t W, size_t O, size_t K_h, size_t K_w,
                         size_t stride, size_t pad, size_t w_batch, int64_t bias_stride_pixel,
                         int64_t bias_stride_channel, int activation, void* stream);
/* nzhip_conv2d_forward with the fp16 image of the weights kept in w_image (see "prepared operands"; NULL:
 * plain nzhip_conv2d_forward). */
int nzhip_conv2d_forward_prepared(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C,
                                  size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                  size_t w_batch, int64_t bias_stride_pixel, int64_t bias_stride_channel, int activation,
                                  nzhip_prepared* w_image, void* stream);

/* Gradient of nzhip_conv2d_forward with respect to x, as one call. In the reference this is the chain
 * Col2ImgNode::backward (src/Nodes.cu:660-665) -> MatMulNode::backward, dA += dC * B^T (:169-182) ->
 * Img2ColNode::backward (:632-640; img2colBackwardKernel, src/OperationKernels.cu:1337-1362):
 *   dx[b][c][h][w] (+)= sum over r, s, o of f16(dy[b][o][ho][wo]) * f16(w_ref[wb][(c,r,s)][o])
 *   with ho * stride = h + pad - r, wo * stride = w + pad - s
 * accumulate != 0 adds into dx (what the chain does), 0 overwrites it. Supported: K_h == K_w, pad <= K_h - 1,
 * stride <= 8; anything else returns NZHIP_E_UNSUPPORTED and the caller runs the chain. With a stride above 1 the
 * call is either one convolution of the zero-filled output gradient or that chain inside the library (column
 * gradient in a pooled workspace), whichever an estimate from the shape finds cheaper; stride-1 layers on images so
 * small that the convolution would write a column matrix itself take the chain too. Same sums either way. */
int nzhip_conv2d_backward_data(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H,
                               size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                               size_t w_batch, int accumulate, void* stream);

/* Gradient of nzhip_conv2d_forward with respect to the weights, as one call. In the reference this is
 * MatMulNode::backward's dB += A^T * dC (src/Nodes.cu:169-182) with A the column matrix that
 * Img2ColNode::forward wrote (:605-630) and dC the pixel-major gradient from Col2ImgNode::backward (:660-665):
 *   dw[wb][(c,r,s)][o] += sum over h, w (and n, for shared weights) of
 *                         f16(x[n][c][h+r-pad][w+s-pad]) * f16(dy[n][o][h][w])
 * Supported: any K_h x K_w of at most 128 taps with stride <= 4 (1x1 is a product on x itself or on its strided
 * pixels); anything else returns NZHIP_E_UNSUPPORTED and the caller runs the chain. Shared weights on images of fewer
 * than 64 output pixels run that chain inside the library as ONE product whose contraction is the pixels of all
 * images (column matrix and transposed gradient in pooled workspaces); same sums either way. */
int nzhip_conv2d_backward_weights(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H,
                                  size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                  size_t w_batch, void* stream);

/* ---- unfused element-wise fallbacks -------------------------------------- */
/* tensorMatrixAdd + MatrixAddKernel (TensorOperations.cuh:785-808, OperationKernels.cu:12-24):
 * out[n][c][:] = a[n or 0][c or 0][:] + b[n or 0][c or 0][:]; h, w must agree, n and c broadcast. */
int nzhip_add_broadcast(float* out, const float* a, const float* b, const size_t shapeOut[4],
                        const size_t shapeA[4], const size_t shapeB[4], void* stream);

/* Tensor::fill (src/Tensor.cu:306-314 -> krnl::Fill, FillKernel, src/OperationKernels.cu:1146-1156):
 * data[0, n) = value, on the device (OutputNode::backward seeds the output gradient with it, src/Nodes.cu:62-66). */
int nzhip_fill(float* data, float value, size_t n, void* stream);

/* nz::data::iRELU (TensorOperations.cuh:19; RectifiedLinearUnitKernel, OperationKernels.cu:230-235). */
int nzhip_relu(float* out, const float* in, size_t n, void* stream);

/* ---- backward of the same path -------------------------------------------- */
/* nz::data::iGEMMBackward (include/NeuZephyr/TensorOperations.cuh:1030-1031, src/TensorOperations.cu:117-120
 * -> krnl::GEMMBackwardParallel, src/OperationKernels.cu:1028-1144): over the batch max(A, B),
 *     C[n or 0][c or 0] += f16(A_nc)[M,K] * f16(B_nc)[K,N]          (M = A.h, K = A.w, N = B.w)
 * i.e. the products are ADDED to what C holds, and a batch dimension in which C has extent 1
 * collects every member (CuttingAndCompress, :873-883). Members are added in a fixed order
 * (the reference's atomicAdd leaves it open). */
int nzhip_gemm_backward(const float* A, const float* B, float* C, const size_t shapeA[4],
                        const size_t shapeB[4], const size_t shapeC[4], void* stream);

/* MatMulNode::backward (src/Nodes.cu:169-182) without the materialised transposes:
 *     dA += dC * B^T        dB += A^T * dC
 * for C = A * B with the forward's shapes and broadcast rules; dA or dB may be NULL to skip it. */
int nzhip_matmul_backward(float* dA, float* dB, const float* A, const float* B, const float* dC,
                          const size_t shapeA[4], const size_t shapeB[4], const size_t shapeC[4], void* stream);

/* ReLUBackwardKernel (src/OperationKernels.cu:242-253): dx = x > 0 ? dy : 0 (overwrites dx). */
int nzhip_relu_backward(float* dx, const float* x, const float* dy, size_t n, void* stream);

/* AddNode::backward for one input (src/Nodes.cu:99-146): equal shapes -> din = dout (copy);
 * otherwise din[n or 0][c or 0][:] += dout[n][c][:] over every (n, c) (gradCopyKernel, :1230-1236). */
int nzhip_add_backward(float* din, const float* dout, const size_t shapeIn[4], const size_t shapeOut[4],
                       void* stream);

/* nz::data::iImg2colBackward (img2colBackwardKernel, src/OperationKernels.cu:1337-1362): every element of the
 * column-matrix gradient is ADDED to the image-gradient element it was copied from. */
int nzhip_im2col_backward(float* dx, const float* dcol, size_t H_out, size_t W_out, size_t C, size_t K_h,
                          size_t K_w, size_t stride, size_t pad, size_t H_in, size_t W_in, size_t batch,
                          void* stream);

/* nz::data::iCol2imgBackward (col2imgBackwardKernel, src/OperationKernels.cu:1384-1402):
 * dcol[b][(h*W_out+w)*C_out + c] = dy[b][c][h][w]. */
int nzhip_col2im_backward(float* dcol, const float* dy, size_t H_out, size_t W_out, size_t C_out,
                          size_t batches, void* stream);

/* ---- fp32-exact matmul and optimizer steps ---------------------------------- */
/* nz::data::tensorGeneralMatrixMul / iGeneralMatrixMul behind Tensor::operator*
 * (include/NeuZephyr/TensorOperations.cuh:998-1019, src/TensorOperations.cu:104-110; GeneralMatrixMulKernel,
 * src/OperationKernels.cu:65-101): C[n][c] = A[n or 0][c or 0] * B[n or 0][c or 0] with NO rounding of
 * the operands, fp32 FMA accumulation in ascending k. M = A.h, N = B.w, K = A.w = B.h. */
int nzhip_matmul_f32(const float* A, const float* B, float* C, const size_t shapeA[4],
                     const size_t shapeB[4], const size_t shapeC[4], void* stream);

/* opt::SGD::step (src/Optimizer.cu:14-19; StochasticGradientDescentKernel, src/OperationKernels.cu:634-640):
 * data -= lr * grad. */
int nzhip_sgd_step(float* data, const float* grad, float lr, size_t n, void* stream);

/* opt::Adam::step (src/Optimizer.cu:86-102; AdamKernel, src/OperationKernels.cu:753-766), t = 1, 2, ...:
 *   m = beta1*m + (1-beta1)*g;  v = beta2*v + (1-beta2)*g*g;
 *   data -= lr * (m / (1-beta1^t)) / (sqrt(v / (1-beta2^t)) + eps)
 * beta^t is evaluated with powf; the reference kernel uses CUDA's approximate __powf, so the last
 * bits of the bias corrections are not pinned by it (its own test compares against std::pow). */
int nzhip_adam_step(float* data, float* m, float* v, const float* grad, float lr, float beta1,
                    float beta2, float eps, int t, size_t n, void* stream);

/* The same steps, and nzhip_fill, for `count` tensors in one launch per NZHIP_MANY_MAX tensors.  No counterpart
 * in the reference, which launches one kernel per parameter (ComputeGraph::update, src/ComputeGraph.cu:541-547;
 * Tensor::zeroGrad, src/Tensor.cu:306-314): the parameters of a small network are a dozen tensors of a few floats
 * each, and a dozen launches cost more than the work.  Every element gets exactly the arithmetic of the one-tensor
 * call (bit-identical results); t[k] is tensor k's step count (Adam counts per call, so the tensors of one update
 * have consecutive counts).  Tensors must not overlap. */
#define NZHIP_MANY_MAX 16
int nzhip_fill_many(int count, float* const* data, const size_t* n, float value, void* stream);
int nzhip_sgd_step_many(int count, float* const* data, const float* const* grad, const size_t* n, float lr, void* stream);
int nzhip_adam_step_many(int count, float* const* data, float* const* m, float* const* v, const float* const* grad,
                         const size_t* n, const int* t, float lr, float beta1, float beta2, float eps, void* stream);

/* ---- softmax (third caller of the GEMM entry: its backward is Jacobian x gradient) --------- */
/* nz::data::Softmax over `batch` contiguous vectors of `len` elements (TensorOperations.cuh:379-392;
 * SummationExpKernel + SoftmaxKernel, src/OperationKernels.cu:477-523): out = exp(in) / sum(exp(in)),
 * no maximum subtracted. exp is the fast hardware form (the reference uses __expf) and the sum is a
 * tree: last bits are not pinned by the reference. */
int nzhip_softmax(float* out, const float* in, size_t len, size_t batch, void* stream);

/* nz::data::softmaxJacobian / iSoftmaxJacobian (TensorOperations.cuh:1091-1106; SoftmaxJacobianKernel,
 * src/OperationKernels.cu:550-565): out[b][x][y] = s_x (1 - s_x) if x == y else -s_x s_y, s = in[b].
 * SoftmaxNode::backward (src/Nodes.cu:538-548) is this followed by nzhip_tensorcore_gemm
 * (J x dY for column vectors, dY x J for row vectors). */
int nzhip_softmax_jacobian(float* out, const float* in, size_t n, size_t batch, void* stream);

/* SoftmaxNode::backward (src/Nodes.cu:538-548) in one kernel, without the n x n Jacobian in memory:
 * dx[b][i] = sum_j fp16(J[b][i][j]) * fp16(dy[b][j]) with J as above, fp32 accumulation in ascending j,
 * i.e. the values nzhip_softmax_jacobian + nzhip_tensorcore_gemm give up to the order of the fp32
 * additions (the Jacobian is symmetric, so column and row vectors are the same sums). dx is overwritten. */
int nzhip_softmax_backward(float* dx, const float* s, const float* dy, size_t n, size_t batch, void* stream);

/* Gradient of the bias parameter of the reference's Conv2d ([1,1,H_out*W_out,O]: per pixel and channel, added to the
 * matmul result): dbias[p*O + o] += sum over n of dz[(n*O + o)*HW + p]. Replaces Col2ImgNode::backward (a transposed
 * copy of the whole gradient) + AddNode::backward (sum over the batch), src/Nodes.cu:660-665, 99-146; the images are
 * added in ascending order onto the value already in dbias, like that chain (which, for a batch of one, copies
 * instead of adding: AddNode::backward with equal shapes; callers keep that case on the two-step path). */
int nzhip_conv2d_backward_bias(float* dbias, const float* dz, size_t N, size_t O, size_t HW, void* stream);

/* The same for a Conv2d followed by ReLU, with ReLUNode::backward (src/Nodes.cu:357-364) in front: writes
 * dz[i] = y[i] > 0 ? dy[i] : 0 over the whole [N,O,HW] gradient and adds its batch sum, transposed, onto dbias in the
 * same pass. dz must not overlap y or dy. */
int nzhip_conv2d_backward_relu_bias(float* dz, float* dbias, const float* y, const float* dy, size_t N, size_t O,
                                    size_t HW, void* stream);

/* ---- the rest of the reference's example network (README.md:62-90): pooling, loss, target expansion ---- */
/* nz::data::iAveragePooling (AveragePoolingKernel, src/OperationKernels.cu:1404-1429; AveragePoolingNode::forward,
 * src/Nodes.cu:678-682): square window, out = mean over the window cells inside the image (cells in the
 * padding do not count), summed row by row, left to right. H_out = (H_in + 2 pad - pool) / stride + 1. */
int nzhip_avgpool2d(float* out, const float* in, size_t pool, size_t stride, size_t pad, size_t batches,
                    size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out, void* stream);

/* nz::data::iAveragePoolingBackward (AveragePoolingBackwardKernel, :1439-1486; AveragePoolingNode::backward,
 * src/Nodes.cu:684-690): din += dout / divisor over every window that covers the element, divisor = pool^2
 * without padding, the number of window cells inside the image with padding. The reference scatters with
 * atomicAdd; here every input element gathers its windows in ascending (row, column) order, the order of a
 * serial run of that scatter. */
int nzhip_avgpool2d_backward(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches,
                             size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out, void* stream);
/* The same with din = instead of din +=: din's old contents are not read. No counterpart in the reference; for the first
 * writer of a gradient that would otherwise be cleared first and then read back as zeros. */
int nzhip_avgpool2d_backward_overwrite(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches,
                                       size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out, void* stream);

/* BinaryCrossEntropyNode::forward (src/Nodes.cu:822-840; BinaryCrossEntropyKernel, src/OperationKernels.cu:648-685):
 * *loss (device memory) = sum_i (-t_i log p_i - (1 - t_i) log(1 - p_i)) / n with the fast hardware logarithm
 * (the reference uses __logf) and a fixed two-level summation order; the reference adds per-block partial sums
 * on the host. Last bits are not pinned by the reference (its test compares at 1e-2). */
int nzhip_bce_loss(float* loss, const float* predict, const float* real, size_t n, void* stream);

/* BinaryCrossEntropyNode::backward (src/Nodes.cu:842-849; BCEBackwardKernel, :692-699):
 * grad_i = ((p_i - t_i) / (p_i (1 - p_i))) / n, overwriting grad. */
int nzhip_bce_backward(float* grad, const float* predict, const float* real, size_t n, void* stream);

/* MeanSquaredErrorNode::forward / backward (src/Nodes.cu:785-811; MeanSquaredErrorKernel, MSEBackwardKernel,
 * src/OperationKernels.cu:579-627): *loss (device memory) = sum_i (p_i - t_i)^2 / n with the summation order of
 * nzhip_bce_loss; grad_i = 2 (p_i - t_i) / n, overwriting grad. */
int nzhip_mse_loss(float* loss, const float* predict, const float* real, size_t n, void* stream);
int nzhip_mse_backward(float* grad, const float* predict, const float* real, size_t n, void* stream);

/* ExpandNode::forward / backward (src/Nodes.cu:585-603; ExpandKernel, CompressKernel, :1282-1301):
 * out[b*n + j] = in[j] for b < batches; and out[j] += sum_b in[b*n + j] in ascending b. */
int nzhip_expand(float* out, const float* in, size_t n, size_t batches, void* stream);
int nzhip_compress(float* out, const float* in, size_t n, size_t batches, void* stream);

/* ---- runtime: device allocator + stream manager -------------------------- */
/* Replace cuStrm::StreamManager<float> (include/NeuZephyr/StreamManager.cuh:131-911) and
 * EventPool (EventPool.cuh:165-457).  One ordered compute stream, nzhip_default_stream(), carries
 * the runtime's copies, memsets and stream-ordered allocations, so producer/consumer order on
 * it needs no per-buffer events.
 *
 * Precondition: the runtime only knows about work on ITS stream.  Memory from nzhip_malloc is
 * handed out, cached and re-issued in the order of that stream, and nzhip_sync_ptr,
 * nzhip_memcpy_* and nzhip_memset are ordered on it.  A caller that passes another stream to a
 * compute entry point whose operands came from nzhip_malloc must call nzhip_stream_wait(stream)
 * before it frees, copies, clears or synchronises those operands through the runtime (and must
 * order the other direction itself, e.g. by synchronising before the compute call).  The nz::
 * C++ layer always computes on nzhip_default_stream() and needs none of this.  Workspaces the
 * library takes internally are tagged with the caller's stream and never migrate. */
void* nzhip_default_stream(void);                 /* the manager's compute stream (hipStream_t) */
int nzhip_malloc(void** ptr, size_t bytes);       /* StreamManager::malloc (:230-240); size in BYTES */
int nzhip_free_async(void* ptr);                  /* StreamManager::freeAsync (:325-335): stream-ordered, cached */
int nzhip_free(void* ptr);                        /* StreamManager::free (:263): blocks until users finished */
/* Page-locked host memory mapped into the device, the storage of nz::data::MappedTensor
 * (src/MappedTensor.cu:88-96: cudaMallocHost; StreamManager::freeHost, StreamManager.cuh:299-302).
 * The pointer is valid on the host and as an operand of every compute entry point; kernels then
 * read and write it over the host link. nzhip_host_free waits for nzhip_default_stream() first. */
int nzhip_host_malloc(void** ptr, size_t bytes);
int nzhip_host_free(void* ptr);
int nzhip_memset(void* ptr, int value, size_t bytes);                 /* :360 */
int nzhip_memcpy_h2d(void* dst, const void* src, size_t bytes);       /* :391, async w.r.t. device */
int nzhip_memcpy_d2d(void* dst, const void* src, size_t bytes);
int nzhip_memcpy_d2h(void* dst, const void* src, size_t bytes);       /* blocks until the copy landed */
/* StreamManager::syncData (:714).  Blocks until nzhip_default_stream() has drained, which covers
 * every piece of work that touches ptr provided the precondition above is kept; ptr itself is
 * not looked at. */
int nzhip_sync_ptr(const void* ptr);
/* StreamManager::streamWait (:840-850), per stream instead of per buffer: everything enqueued
 * later on nzhip_default_stream() (frees and the re-issue of freed blocks, copies, memsets,
 * kernels) runs after everything enqueued so far on `stream`.  Does not block the host. */
int nzhip_stream_wait(void* stream);
int nzhip_sync_all(void);                         /* StreamManager::sync (:671) */
/* allocator statistics (bytes handed out, bytes cached, hipMalloc calls so far) */
int nzhip_allocator_stats(size_t* bytes_in_use, size_t* bytes_cached, size_t* device_allocs);
int nzhip_allocator_trim(void);                   /* return cached blocks to the driver */

#ifdef __cplusplus
}
#endif
#endif /* NZHIP_H */
