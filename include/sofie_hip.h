/*
 * sofie_hip.h -- C ABI of the MI355X (gfx950) kernel library that SOFIE-generated
 * inference code calls instead of a host BLAS.
 *
 * The generated code of the reference calls, per operator, the Fortran BLAS routines
 * declared in its own header (src/SOFIE_core/src/RModel_Base.cxx:40-58: sgemm_, sgemv_,
 * saxpy_, scopy_) plus the header templates SOFIE::UTILITY::Im2col and
 * UnidirectionalBroadcast (src/SOFIE_core/inc/SOFIE/SOFIE_common.hxx:346-518) on host
 * pointers. Each entry point below names the emitted call sequence it replaces.
 *
 * Conventions
 *  - Every tensor pointer is a DEVICE pointer unless the name says host.
 *  - All matrices are row-major with explicit leading dimensions in ELEMENTS; no
 *    column-major swap trick is needed by the caller.
 *  - Calls are asynchronous on the context's stream; sofie_hip_sync() waits.
 *  - Return value: 0 on success, a negative SOFIE_HIP_E* code otherwise;
 *    sofie_hip_last_error() gives the message. Generated code turns a non-zero
 *    status into std::runtime_error, the reference's error convention
 *    (ROperator_Gemm.hxx:76,143,295,347).
 *  - The library keeps no global mutable state apart from the per-GPU scratch array of
 *    sofie_hip_qgemm_s8_noalloc; one context per Session, one Session per thread slot
 *    (the reference's threading contract, SOFIEHelpers.hxx:27-48).
 */
#ifndef SOFIE_HIP_H
#define SOFIE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct sofie_hip_ctx sofie_hip_ctx;

enum {
   SOFIE_HIP_OK = 0,
   SOFIE_HIP_EINVAL = -1,       /* bad argument (null pointer, negative size, bad enum) */
   SOFIE_HIP_EHIP = -2,         /* a HIP runtime call failed */
   SOFIE_HIP_ENOMEM = -3,       /* device allocation failed */
   SOFIE_HIP_EUNSUPPORTED = -4  /* valid request that no kernel covers */
};

/* Fused activation of an epilogue. Only ReLU exists, as in the reference
 * (ROperator_Gemm.hxx:377-381 acts on EActivationType::RELU only). */
enum { SOFIE_ACT_NONE = 0, SOFIE_ACT_RELU = 1 };

/* How the fp32 bias operand of sofie_hip_gemm_f32 is shaped. */
enum {
   SOFIE_BIAS_NONE = 0,
   SOFIE_BIAS_ROW = 1,  /* [N]: one value per output column, same for every row */
   SOFIE_BIAS_FULL = 2, /* [M,N] with leading dimension ldy: already broadcast */
   SOFIE_BIAS_COL = 3   /* [M]: one value per output row */
};

/* Element type written by the quantized / FP8 GEMMs. */
enum {
   SOFIE_OUT_S8 = 0,   /* requantised int8 */
   SOFIE_OUT_F32 = 1,  /* fp32 */
   SOFIE_OUT_S32 = 2,  /* raw int32 accumulators (+bias) */
   SOFIE_OUT_BF16 = 3  /* bfloat16, round to nearest even */
};

/* Memory layout of an int8 activation tensor. */
enum { SOFIE_LAYOUT_NCHW = 0, SOFIE_LAYOUT_NHWC = 1 };

/* ---------------------------------------------------------------- context, memory */

/* Create a context on `device`. `stream` is a hipStream_t to launch on (borrowed), or
 * NULL to create and own a new stream. Replaces nothing in the reference: its Session
 * owns host vectors only (RModel.cxx:574-653). */
int sofie_hip_create(sofie_hip_ctx **ctx, int device, void *stream);
int sofie_hip_destroy(sofie_hip_ctx *ctx);
/* Message of the last failed call on this context ("" if none). Never NULL. */
/* A promise of the caller: the weight tensors handed to the convolution entry points of this context from now on do
 * not change (and their memory is not freed and reused) while the context lives or until the promise is taken back
 * with on = 0. The library then keeps the copy of a weight tensor that it lays out for its kernels
 * (sofie_hip_conv2d_f32: [K][channel]; sofie_hip_conv_transpose2d_f32: the gathered sub-kernels of the output phases)
 * in a buffer of its own per tensor and geometry, made by the first call, instead of making it in front of every
 * launch in the scratch buffer; at most SOFIE_HIP_PACKED_MAX tensors, later ones are laid out per call as before.
 * on = 0 frees the copies. Not allowed while a graph is recorded; a new tensor met while a graph is recorded is laid
 * out per call. A generated Session makes the promise in its constructor: its weights are uploaded once and never
 * written again. The reference re-lays a Conv's weights inside every infer call (ROperator_Conv.hxx:342-362); no
 * counterpart of the promise exists there. */
#define SOFIE_HIP_PACKED_MAX 256
int sofie_hip_constant_weights(sofie_hip_ctx *ctx, int on);

const char *sofie_hip_last_error(const sofie_hip_ctx *ctx);
/* ABI version of the library (bumped on incompatible change). */
int sofie_hip_version(void);

/* Device allocations owned by the caller (the generated Session): weights uploaded once
 * in its constructor and the intermediate-tensor arena. Replace the std::vector<float>
 * members and `new char[]` pool of the generated Session (RModel.cxx:574-604). */
int sofie_hip_malloc(sofie_hip_ctx *ctx, void **dptr, size_t bytes);
int sofie_hip_free(sofie_hip_ctx *ctx, void *dptr);
/* Page-locked host memory for inputs and outputs: an upload from (download into) it runs at the rate of the link,
 * without the driver's staging copy of pageable memory. The generated Session hands such a buffer out per input
 * (pinned_input_<name>()); infer() on that pointer is then bound by PCIe, not by the copy. No counterpart in the
 * reference (its Session reads the caller's host pointer directly, RModel.cxx:680-801). */
int sofie_hip_host_malloc(sofie_hip_ctx *ctx, void **hptr, size_t bytes);
int sofie_hip_host_free(sofie_hip_ctx *ctx, void *hptr);
int sofie_hip_upload(sofie_hip_ctx *ctx, void *dst_device, const void *src_host, size_t bytes);
int sofie_hip_download(sofie_hip_ctx *ctx, void *dst_host, const void *src_device, size_t bytes);
int sofie_hip_copy(sofie_hip_ctx *ctx, void *dst_device, const void *src_device, size_t bytes);
int sofie_hip_memset(sofie_hip_ctx *ctx, void *dptr, int byte_value, size_t bytes);
int sofie_hip_sync(sofie_hip_ctx *ctx);

/* HIP graph of a fixed call sequence. Between capture_begin and capture_end the calls made on the context are
 * recorded instead of run; graph_launch replays them with one launch (a launch-bound chain of small kernels, such
 * as a small MLP, then costs one submission instead of one per operator). The recorded calls keep their
 * pointer arguments. Nothing may allocate while recording: run the sequence once eagerly first, so that the
 * context's scratch buffer has its final size (a call that would grow it fails with a message saying so).
 * Between begin and end sofie_hip_malloc, _free, _upload, _download, _memset, _sync, _timer_start, _timer_stop and
 * _graph_destroy return SOFIE_HIP_EINVAL and do nothing (they would wait on, or record a memset node into, the
 * capturing stream). capture_end with a NULL result pointer abandons the recording. A recorded graph keeps the
 * address of the context's scratch buffer: until it is destroyed, a later call on the same context that needs a
 * larger scratch buffer fails with SOFIE_HIP_EINVAL instead of freeing the buffer under the graph. No counterpart
 * in the reference (its generated code is a CPU call sequence). */
typedef struct sofie_hip_graph sofie_hip_graph;
int sofie_hip_capture_begin(sofie_hip_ctx *ctx);
int sofie_hip_capture_end(sofie_hip_ctx *ctx, sofie_hip_graph **graph);
int sofie_hip_graph_launch(sofie_hip_ctx *ctx, sofie_hip_graph *graph);
int sofie_hip_graph_destroy(sofie_hip_ctx *ctx, sofie_hip_graph *graph);

/* Event timing on the context's stream: start, enqueue work, stop (synchronises). */
int sofie_hip_timer_start(sofie_hip_ctx *ctx);
int sofie_hip_timer_stop(sofie_hip_ctx *ctx, float *elapsed_ms);

/* Per-launch timing of whatever is enqueued on the context between the two calls: trace_begin records an event,
 * every kernel launch of the library on this context then records one behind itself, and trace_end waits for the
 * stream and writes one line per launch, in launch order, "<kernel> <microseconds>\n": the time from the end of the
 * launch before it (or from trace_begin) to its own end, so the lines of a sequence add up to the sequence's time on
 * the device, the gaps between dependent kernels included. The text is truncated to `capacity` bytes (always
 * NUL-terminated); *launches receives the number of launches seen. Not allowed while a graph is being recorded; at
 * most SOFIE_HIP_TRACE_MAX launches are kept, later ones are counted but not timed. No counterpart in the reference
 * (its generated code is timed from outside); it is what the benchmark reports per-kernel figures of a Session from. */
#define SOFIE_HIP_TRACE_MAX 4096
int sofie_hip_trace_begin(sofie_hip_ctx *ctx);
int sofie_hip_trace_end(sofie_hip_ctx *ctx, char *text, size_t capacity, int *launches);

/* ---------------------------------------------------------------- fp32 operators */

/* Y[M,N] = alpha * op(A) * op(B) + beta * bias, then optional ReLU.
 * op(A) is [M,K]: A is stored [M,K] (lda >= K) or, if transA, [K,M] (lda >= M).
 * op(B) is [K,N]: B is stored [K,N] (ldb >= N) or, if transB, [N,K] (ldb >= K).
 * bias == NULL requires beta == 0 (error otherwise, as ROperator_Gemm.hxx:343-349).
 * Replaces the emitted sequence std::copy(bias_bcast -> Y); BLAS::sgemm_(...); ReLU loop
 * of ROperator_Gemm<float>::Generate (ROperator_Gemm.hxx:360-381) and the bias
 * materialisation of GenerateInitCode (:271-290): a rank-1 bias is broadcast inside
 * the kernel epilogue instead of being stored M times. */
int sofie_hip_gemm_f32(sofie_hip_ctx *ctx, int transA, int transB, int M, int N, int K,
                       float alpha, const float *A, int lda, const float *B, int ldb,
                       float beta, const float *bias, int bias_kind, float *Y, int ldy,
                       int act);

/* A chain of fully connected layers in one launch:
 *   a_0 = x [M, dims[0]];  a_l = act_l(a_{l-1} * W_l + bias_l), l = 1..n_layers;  y = a_{n_layers} [M, dims[n_layers]]
 * W[l-1] is [dims[l-1], dims[l]] row-major (the operand B of a Gemm with transB = 0), bias[l-1] one row of dims[l]
 * values or NULL (bias itself may be NULL), act[l-1] SOFIE_ACT_NONE or SOFIE_ACT_RELU. Replaces n_layers times the
 * sequence the reference emits per Gemm (ROperator_Gemm.hxx:292-390: bias copy, BLAS::sgemm_, ReLU loop) when every
 * layer is small (widths up to SOFIE_MLP_MAX_WIDTH): the intermediate activations never leave the chip and the
 * chain costs one launch. The emitter joins Gemm operators into such a call when each one's output feeds only the
 * next (RModel::FuseGemmChain). Sums are fp32 fused multiply-adds over k in increasing order within a part of K;
 * the result agrees with the separate calls to the usual 1e-5 relative tolerance, not bit for bit. */
#define SOFIE_MLP_MAX_LAYERS 16
#define SOFIE_MLP_MAX_WIDTH 1024
int sofie_hip_mlp_f32(sofie_hip_ctx *ctx, int n_layers, const int *dims, const float *const *W,
                      const float *const *bias, const int *act, const float *x, int ldx, float *y, int ldy,
                      int M);

/* Stacked matrix products (numpy.matmul on operands of rank > 2) in one launch:
 *   Y[i] = alpha * op(A[ia(i)]) * op(B[ib(i)]), optional ReLU, for every index i of the n_lead leading dimensions
 * lead[0..n_lead) (row-major, last dimension fastest). stride_a[d] / stride_b[d] are the element strides of A / B
 * along leading dimension d, 0 where the operand has extent 1 there and is broadcast; Y is dense: product i
 * starts M * ldy elements after product i - 1. Replaces the loop over the stack that the reference emits around
 * BLAS::sgemm_ (ROperator_Gemm.hxx:353-387), which hands every iteration the first matrices of A and B; here
 * each product reads its own. No bias (the emitter refuses one on stacked operands). */
#define SOFIE_GEMM_MAX_LEAD 6
int sofie_hip_gemm_f32_stacked(sofie_hip_ctx *ctx, int transA, int transB, int M, int N, int K, float alpha,
                               const float *A, int lda, const float *B, int ldb, float *Y, int ldy, int n_lead,
                               const int *lead, const long long *stride_a, const long long *stride_b, int act);

/* NCHW 2-D convolution y = conv(x, w) + bias[oc], optional ReLU.
 * x [N,C,H,W], w [OC, C/groups, KH, KW] (the ONNX layout, unpacked), bias [OC] or NULL,
 * y [N,OC,OH,OW] with OH = (H + pad_top + pad_bottom - (dil_h*(KH-1)+1)) / stride_h + 1 (pads in ONNX order:
 * top, left, bottom, right; begin and end pads may differ, as auto_pad SAME_UPPER / SAME_LOWER make them).
 * Replaces, per image, the emitted weight re-layout loop, UTILITY::Im2col, BLAS::sgemm_
 * and BLAS::saxpy_ of ROperator_Conv<float>::Generate (ROperator_Conv.hxx:342-518) and
 * the following ROperator_Relu loop (ROperator_Relu.hxx:54-66) with one implicit-GEMM
 * kernel over the whole batch; no im2col matrix is materialised. */
int sofie_hip_conv2d_f32(sofie_hip_ctx *ctx, const float *x, const float *w,
                         const float *bias, float *y, int N, int C, int H, int W, int OC,
                         int KH, int KW, int pad_top, int pad_left, int pad_bottom, int pad_right,
                         int stride_h, int stride_w, int dil_h, int dil_w, int groups, int act);

/* NCDHW 3-D convolution y = conv(x, w) + bias[oc], optional ReLU.
 * x [N,C,D,H,W], w [OC, C/groups, KD, KH, KW], bias [OC] or NULL, y [N,OC,OD,OH,OW] with
 * OD = (D + 2*pad_d - (dil_d*(KD-1)+1)) / stride_d + 1 (same for H, W). Replaces, per image (and group), the
 * emitted UTILITY::Im2col_3d, BLAS::sgemm_ and BLAS::saxpy_ of ROperator_Conv<float>::Generate for fDim == 3
 * (ROperator_Conv.hxx:432-451,499-518; SOFIE_common.hxx:522-580). The sum of an output runs over
 * (channel, kd, kh, kw) in this order, one rounded product and one rounded addition per term. */
int sofie_hip_conv3d_f32(sofie_hip_ctx *ctx, const float *x, const float *w,
                         const float *bias, float *y, int N, int C, int D, int H, int W, int OC,
                         int KD, int KH, int KW, int pad_d, int pad_h, int pad_w, int stride_d,
                         int stride_h, int stride_w, int dil_d, int dil_h, int dil_w, int groups,
                         int act);

/* NCHW 2-D transposed convolution (ONNX ConvTranspose), optional ReLU.
 * x [N,C,H,W], w [C, OC/groups, KH, KW] (the ONNX layout), bias [OC] or NULL, y [N,OC,OH,OW]:
 *   y[n,oc,oy,ox] = bias[oc] + sum over (ic,kh,kw) with oy + pad_h - kh*dil_h = stride_h*iy (same for x)
 *                   of x[n,ic,iy,ix] * w[ic,oc',kh,kw].
 * OH and OW are given by the caller: stride*(in-1) + dil*(K-1) + 1 + output_padding - pad_begin - pad_end
 * (ROperator_ConvTranspose.icc:83-90); pad_h / pad_w are the begin pads. Replaces the emitted kernel
 * re-layout, BLAS::sgemm_ into the column matrix, UTILITY::col2im and BLAS::saxpy_ of
 * ROperator_ConvTranspose<float>::Generate (ROperator_ConvTranspose.icc:232-474) with the implicit-GEMM
 * convolution kernel: per output phase (oy mod stride, ox mod stride) the reversed taps that
 * reach it (up to four phases share one launch), or, with a dilation, one launch over the zero-interleaved input; no column matrix exists. */
int sofie_hip_conv_transpose2d_f32(sofie_hip_ctx *ctx, const float *x, const float *w,
                                   const float *bias, float *y, int N, int C, int H, int W,
                                   int OC, int KH, int KW, int pad_h, int pad_w, int stride_h,
                                   int stride_w, int dil_h, int dil_w, int groups, int OH, int OW,
                                   int act);

/* Inference BatchNormalization on [N, C, plane] (plane = H*W, or 1 for a [N,C] tensor):
 * y = (x - mean[c]) * scale[c] + bias[c], optional ReLU, where scale[c] already holds
 * gamma[c] / sqrt(var[c] + epsilon) (the emitter folds it, as the reference's Initialize does,
 * ROperator_BatchNormalization.hxx:163-167). Replaces the emitted BLAS::scopy_, BLAS::saxpy_(-mean), the
 * multiply loop, BLAS::saxpy_(+bias) and the ReLU loop of ROperator_BatchNormalization<float>::Generate
 * (:196-226), and the four [N,C,H,W]-sized broadcast tensors they read, with one pass over x. */
int sofie_hip_batchnorm_f32(sofie_hip_ctx *ctx, const float *x, const float *scale, const float *mean,
                            const float *bias, float *y, int N, int C, int plane, int act);

/* Einstein summation of n_inputs fp32 operands that is not a matrix product:
 *   y[o0, o1, ...] = sum over s0, s1, ... of x_0[...] * x_1[...] * ...
 * The n_labels labels are numbered with the n_out output labels first, in the order of y's dimensions (y is
 * dense row-major over them), then the summed labels, the first of them the outermost loop. extent[l] is the
 * size of label l; stride[i * n_labels + l] is operand i's element stride along label l, 0 where the operand
 * does not carry the label (a repeated label adds its strides up). Products and sums are rounded one by one in
 * loop order, as in the nest of host loops that ROperator_Einsum<float>::Generate emits for the general case
 * (ROperator_Einsum.hxx:236-278), which this call replaces. Equations that are (stacked) matrix products are
 * emitted as sofie_hip_gemm_f32 calls instead, where the reference emits BLAS::sgemm_ (:280-336). */
#define SOFIE_EINSUM_MAX_INPUTS 4
#define SOFIE_EINSUM_MAX_LABELS 12
int sofie_hip_einsum_f32(sofie_hip_ctx *ctx, int n_inputs, const float *const *inputs, int n_labels, int n_out,
                         const int *extent, const long long *stride, float *y);

/* y[i] = x[i] > 0 ? x[i] : 0. Replaces the loop of ROperator_Relu.hxx:62-64. */
int sofie_hip_relu_f32(sofie_hip_ctx *ctx, const float *x, float *y, size_t len);

/* NCHW max pooling over NC = N*C planes; pads in ONNX order (top, left, bottom, right);
 * floor output size; padding cells never win. Replaces the emitted loops of
 * ROperator_Pool.hxx:371-416. */
int sofie_hip_maxpool2d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, int H,
                            int W, int kh, int kw, int pad_t, int pad_l, int pad_b,
                            int pad_r, int stride_h, int stride_w);

/* NCHW average pooling over NC = N*C planes, same geometry rules as the max pooling. A window's values are summed
 * in row-major order and divided once by the number of cells: those inside the image, or kh*kw when
 * count_include_pad is set. GlobalAveragePool is the call with kh = H, kw = W, no pads, stride 1. Replaces the
 * emitted loops of ROperator_Pool.hxx:371-416 in AveragePool mode (sum, nsum, `value /= float(nsum)`). */
int sofie_hip_avgpool2d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, int H, int W,
                            int kh, int kw, int pad_t, int pad_l, int pad_b, int pad_r, int stride_h,
                            int stride_w, int count_include_pad);

/* Max and average pooling over three spatial axes, [NC][dims[0]][dims[1]][dims[2]] fp32: kernel[3], strides[3],
 * pads[6] in ONNX order (the three begin pads, then the three end pads), floor output size, the window walked in
 * row-major order with cells outside the volume skipped (for the average: summed, then divided once by the cells
 * inside the volume, or by the whole window with count_include_pad). Replaces the emitted loops of
 * ROperator_Pool.hxx:417-470 (the fDim == 3 branch). A pooling over one spatial axis (ROperator_Pool.hxx:329-370) is
 * the 2-D call with H = 1 and a 1 x k kernel. */
int sofie_hip_maxpool3d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, const int *dims,
                            const int *kernel, const int *pads, const int *strides);
int sofie_hip_avgpool3d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, const int *dims,
                            const int *kernel, const int *pads, const int *strides,
                            int count_include_pad);

/* ---------------------------------------------------------------- quantized operators
 * The reference has no quantized operator (its parser rejects int8 initialisers,
 * src/SOFIE_parsers/src/RModelParser_ONNX.cxx:560-591); these follow ONNX's
 * QuantizeLinear / DequantizeLinear / QLinearMatMul / QLinearConv and are emitted through
 * the same ROperator interface. Requantisation is one fixed formula everywhere:
 *     r = rint_half_even( float(acc + bias) * scale[channel] )
 *     q = clamp(r + zp_y, lo, 127),  lo = (act == RELU) ? max(zp_y, -128) : -128        */

/* q = sat_s8(rint_half_even(x / scale) + zp). */
int sofie_hip_quantize_f32_s8(sofie_hip_ctx *ctx, const float *x, int8_t *q, size_t len,
                              float scale, int zp);
/* x = (q - zp) * scale. */
int sofie_hip_dequantize_s8_f32(sofie_hip_ctx *ctx, const int8_t *q, float *x, size_t len,
                                float scale, int zp);

/* int8 GEMM with int32 accumulation: acc[m,n] = sum_k A[m,k] * B[k,n] (+ bias[n]).
 * A [M,K] row-major (lda); B [K,N] row-major (ldb) or, if transB, [N,K].
 * scale [N] fp32 per output column (= s_a*s_b[n]/s_y), bias [N] int32 or NULL.
 * A's zero-point is folded by the caller: bias[n] -= zp_a * sum_k B[k,n].
 * out_kind: SOFIE_OUT_S8 (requantised, zp_y, act), SOFIE_OUT_F32 (float(acc)*scale[n],
 * act), SOFIE_OUT_S32 (acc+bias; scale may be NULL). ldy in elements of the output type. */
int sofie_hip_qgemm_s8(sofie_hip_ctx *ctx, int transB, int M, int N, int K, const int8_t *A,
                       int lda, const int8_t *B, int ldb, const float *scale,
                       const int32_t *bias, int zp_y, int act, void *Y, int ldy, int out_kind);

/* Two QLinearMatMul layers, the second one narrow (a classifier's last two fully connected layers), in one call:
 *   T = sofie_hip_qgemm_s8(transB = 1, A [M,K], B1 [N1,K], scale1, bias1, zp_mid, act1) -> int8 [M,N1]
 *   Y = sofie_hip_qgemm_s8(transB = 1, T, B2 [N2,N1], scale2, bias2, zp_y, act2, out_kind)  (S8 or F32)
 * with exactly those results. `mid` [M, ldmid] is a tensor the call may use for T; what it holds afterwards is
 * unspecified. When the first layer's K is long enough to be cut into slices and N2 <= 8, the pass that adds the
 * slices' partial sums also applies the second layer and T is never written (one kernel and one pass over memory
 * less); otherwise the call is the two calls above through `mid`. The emitter joins two QLinearMatMul operators
 * into this call when the first one's output feeds only the second (RModel::FuseQLinearPair). Replaces two of the
 * reference's emitted Gemm sequences (ROperator_Gemm.hxx:292-390) on dequantised tensors. */
int sofie_hip_qgemm_s8_pair(sofie_hip_ctx *ctx, int M, int K, const int8_t *A, int lda, int N1, const int8_t *B1,
                            int ldb1, const float *scale1, const int32_t *bias1, int zp_mid, int act1,
                            int8_t *mid, int ldmid, int N2, const int8_t *B2, int ldb2, const float *scale2,
                            const int32_t *bias2, int zp_y, int act2, void *Y, int ldy, int out_kind);

/* sofie_hip_qgemm_s8 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments, same kernels, same results bit for bit, but the call
 * never allocates or frees. It has no counterpart in the reference. The two paths of sofie_hip_qgemm_s8 that use
 * memory beyond the operands (the int32 partial sums of a long K cut into slices; the transposed copy of a
 * B [K,N] whose leading dimension is not a multiple of 16) take it from a fixed array of
 * SOFIE_HIP_NOALLOC_SCRATCH_BYTES that the library holds on every GPU it runs on until the process ends; a shape
 * that needs more returns SOFIE_HIP_EINVAL with a message and launches nothing (splits * M * round_up(N, 4) * 4
 * bytes for the K slices, at most 16 slices; N * K bytes for the copy). All calls on one GPU share that array:
 * the library lets them use it in turns (each call's kernels wait, on the device, for an event recorded behind the
 * kernels of the call before it, whatever context, stream or thread that call came from), so calls from several
 * contexts give the right results and run one after the other. Only calls recorded into a HIP graph are outside
 * that order: a recorded call must not overlap with other no-allocation calls on the same GPU. Nothing in the array
 * has to start at zero: every word whose value is used has been written by the same call. */
#define SOFIE_HIP_NOALLOC_SCRATCH_BYTES (32u << 20)
int sofie_hip_qgemm_s8_noalloc(sofie_hip_ctx *ctx, int transB, int M, int N, int K, const int8_t *A,
                               int lda, const int8_t *B, int ldb, const float *scale,
                               const int32_t *bias, int zp_y, int act, void *Y, int ldy, int out_kind);

/* int8 2-D convolution with int32 accumulation and fused requantisation.
 * x, y: int8 activations in x_layout / y_layout. w int8 (symmetric, zero-point 0):
 * w_layout SOFIE_LAYOUT_NCHW = ONNX [OC, C/groups, KH, KW], SOFIE_LAYOUT_NHWC =
 * [OC, KH, KW, C/groups] (channels innermost, the order the matrix-core kernel reads).
 * bias [OC] int32 or NULL; scale [OC] fp32.
 * Pads in ONNX order (top, left, bottom, right; begin and end pads may differ). Padding cells hold zp_x (so
 * that they contribute zero once the caller has folded bias[oc] -= zp_x * sum(w[oc])). out_kind SOFIE_OUT_S8 or SOFIE_OUT_S32.
 * The matrix-core kernel takes groups = 1, C % 32 == 0, OC % 64 == 0 with every layout NHWC;
 * NCHW operands of such a shape are converted through the context's scratch buffer on each
 * call, every other shape runs a plain one-thread-per-output kernel. */
int sofie_hip_qconv2d_s8(sofie_hip_ctx *ctx, const int8_t *x, int x_layout, const int8_t *w,
                         int w_layout, const int32_t *bias, const float *scale, void *y,
                         int y_layout, int N, int C, int H, int W, int OC, int KH, int KW,
                         int pad_top, int pad_left, int pad_bottom, int pad_right, int stride_h,
                         int stride_w, int groups, int zp_x, int zp_y, int act, int out_kind);

/* QLinearConv -> (ReLU) -> MaxPool in one call: y is the pooled int8 tensor
 * [N, OC, PH, PW] (y_layout), PH = (OH - pool_kh) / pool_stride_h + 1, no pooling pads.
 * Same operands and rules as sofie_hip_qconv2d_s8; the result equals that call followed by
 * sofie_hip_maxpool2d_s8 bit for bit. One-input-channel 3x3 layers with 2x2/2 pooling run a
 * single kernel that never writes the unpooled tensor; other shapes run the convolution
 * into the context's scratch buffer and pool from there. Replaces the reference's Conv,
 * Relu and MaxPool emissions (ROperator_Conv.hxx:302-522, ROperator_Relu.hxx:54-66,
 * ROperator_Pool.hxx:371-416) for quantized tensors. */
int sofie_hip_qconv2d_pool_s8(sofie_hip_ctx *ctx, const int8_t *x, int x_layout, const int8_t *w,
                              int w_layout, const int32_t *bias, const float *scale, int8_t *y,
                              int y_layout, int N, int C, int H, int W, int OC, int KH, int KW,
                              int pad_top, int pad_left, int pad_bottom, int pad_right, int stride_h,
                              int stride_w, int groups, int zp_x, int zp_y, int act, int pool_kh,
                              int pool_kw, int pool_stride_h, int pool_stride_w);

/* A chain of QLinearConv layers in one call: layer 0 reads x, every later layer the output of the layer before it
 * (layers[l].y in layers[l].y_layout); each layer is what sofie_hip_qconv2d_s8 (pool_kh == 0) or
 * sofie_hip_qconv2d_pool_s8 computes, int8 out, and the results are bit-identical to those calls made one after the
 * other. What the call adds: two consecutive 3x3 stride-1 layers on 32 or 64 channels run as ONE kernel launch when
 * every workgroup owns the same whole images in both (the batch a multiple of the workgroups, as at batch 4096): a
 * workgroup then reads in the second layer only what it wrote itself in the first, so no kernel boundary is needed
 * between them. Other shapes run layer by layer. Replaces the emitted Conv sequences of consecutive Conv (+ Relu,
 * + MaxPool) operators (ROperator_Conv.hxx:377-522, ROperator_Pool.hxx:371-416), each of which ends with its whole
 * output in host memory before the next begins. */
#define SOFIE_QCONV_CHAIN_MAX 8
typedef struct sofie_hip_qconv_layer {
   const int8_t *w;            /* weights, layout w_layout */
   int w_layout;
   const int32_t *bias;        /* [OC] or NULL */
   const float *scale;         /* [OC] */
   int8_t *y;                  /* the layer's (pooled) output */
   int y_layout;
   int C, H, W, OC, KH, KW;    /* input channels and size, output channels, kernel */
   int pad_top, pad_left, pad_bottom, pad_right, stride_h, stride_w, groups;
   int zp_x, zp_y, act;
   int pool_kh, pool_kw, pool_stride_h, pool_stride_w;   /* fused max pooling behind the activation; pool_kh == 0: none */
} sofie_hip_qconv_layer;
int sofie_hip_qconv2d_s8_chain(sofie_hip_ctx *ctx, const int8_t *x, int x_layout, int N, int n_layers,
                               const sofie_hip_qconv_layer *layers);

/* QuantizeLinear -> QLinearConv -> (ReLU) -> (MaxPool) in one call, for the first layer of a
 * quantized network: x is the float tensor [N, C, H, W], quantized as in
 * sofie_hip_quantize_f32_s8(x, x_scale, zp_x); everything else as in
 * sofie_hip_qconv2d_pool_s8, pool_kh = pool_kw = 0 meaning no pooling. One-input-channel 3x3
 * stride-1 pad-1 layers quantize while the image is copied on chip and never write the int8
 * input; other shapes quantize into the context's scratch buffer first. Bit-identical to the
 * separate calls. */
int sofie_hip_quantize_qconv2d_s8(sofie_hip_ctx *ctx, const float *x, float x_scale, int zp_x,
                                  const int8_t *w, int w_layout, const int32_t *bias,
                                  const float *scale, int8_t *y, int y_layout, int N, int C, int H,
                                  int W, int OC, int KH, int KW, int pad_top, int pad_left, int pad_bottom,
                                  int pad_right, int stride_h, int stride_w, int groups, int zp_y, int act,
                                  int pool_kh, int pool_kw, int pool_stride_h, int pool_stride_w);

/* int8 max pooling, NCHW or NHWC. */
int sofie_hip_maxpool2d_s8(sofie_hip_ctx *ctx, const int8_t *x, int8_t *y, int layout, int N,
                           int C, int H, int W, int kh, int kw, int pad_t, int pad_l,
                           int pad_b, int pad_r, int stride_h, int stride_w);

/* Layout change of an int8 activation tensor [N,C,H,W] <-> [N,H,W,C]. */
int sofie_hip_relayout_s8(sofie_hip_ctx *ctx, const int8_t *x, int8_t *y, int N, int C, int H,
                          int W, int from_layout, int to_layout);

/* One-byte-element matrix transpose: src [rows, cols] (ld_src) -> dst [cols, rows] (ld_dst).
 * Used once per weight tensor by a Session constructor to bring an ONNX [K,N] int8 / e4m3
 * matrix into the K-contiguous [N,K] layout the GEMM kernels read fastest (then transB = 1);
 * the reference re-lays weights out on every infer call instead (ROperator_Conv.hxx:342-363).
 * rows % 16 == 0, cols % 4 == 0, ld_src % 4 == 0, ld_dst % 16 == 0. */
int sofie_hip_transpose_bytes(sofie_hip_ctx *ctx, const void *src, void *dst, int rows, int cols,
                              int ld_src, int ld_dst);

/* FP8 e4m3 (OCP e4m3fn) GEMM with fp32 accumulation:
 *   t = (sum_k a*b) * (scale_a*scale_b) [+ bias[n]]  -> bf16 (RNE) or fp32.
 * A [M,K] row-major; B [K,N] row-major or, if transB, [N,K]; bias [N] fp32 or NULL. */
int sofie_hip_gemm_fp8(sofie_hip_ctx *ctx, int transB, int M, int N, int K, const uint8_t *A,
                       int lda, const uint8_t *B, int ldb, float scale_a, float scale_b,
                       const float *bias, void *Y, int ldy, int out_kind);

/* fp32 -> e4m3 codes of x * inv_scale, RNE, saturating at +-448 (per-tensor scaling). */
int sofie_hip_quantize_f32_e4m3(sofie_hip_ctx *ctx, const float *x, uint8_t *q, size_t len,
                                float inv_scale);

#ifdef __cplusplus
}
#endif
#endif /* SOFIE_HIP_H */
