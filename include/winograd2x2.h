/*
 * C ABI of the MI355X (gfx950) Winograd F(2x2,3x3) forward ops.
 *
 * Plain pointers and sizes only.  Every device pointer is owned by the caller; no
 * entry point allocates or frees device memory or synchronises: work is queued on
 * `stream` (a hipStream_t passed as void*; NULL is the null stream) and the call
 * returns.  Calls are re-entrant and thread-safe, and keep no state between calls
 * (the two exceptions say so: swc_winograd2x2_conv_grad_static shares one fixed
 * scratch array per GPU, swc_winograd2x2_conv_force_tiling sets a per-thread choice).
 *
 * Citations name the interface of the reference (xingyul/sparse-winograd-cnn) that
 * each entry point stands in for; paths are relative to the reference checkout.
 */
#ifndef WINOGRAD2X2_H_
#define WINOGRAD2X2_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *swc_stream_t;

/* Exported from the shared library; everything else in it is hidden. */
#define SWC_API __attribute__((visibility("default")))

/* Status codes: 0 on success, negative on error.  Nothing here calls exit(). */
#define SWC_OK 0
#define SWC_ERR_NULL_POINTER (-1) /* a required pointer is NULL */
#define SWC_ERR_BAD_DIMS (-2)     /* a dimension is <= 0, inconsistent, or too large to index */
#define SWC_ERR_BAD_PAD (-3)      /* pad_h/pad_w other than 1: the only geometry the ops define */
#define SWC_ERR_HIP (-4)          /* the HIP runtime refused the launch; see swc_last_hip_error() */
#define SWC_ERR_BAD_RANK (-5)     /* op-level wrappers: wrong tensor rank or leading dimension */
#define SWC_ERR_UNSUPPORTED (-6)  /* valid arguments that this entry point has no kernel for (see its comment) */
#define SWC_ERR_TOO_LARGE (-7)    /* valid arguments that need more than this entry point's fixed scratch memory */

SWC_API const char *swc_strerror(int status);
/* hipError_t of the most recent failed launch on the calling thread (0 if none). */
SWC_API int swc_last_hip_error(void);
/* Library version, "major.minor". */
SWC_API const char *swc_version(void);
/* Diagnostic with no counterpart in the reference: the name of the convolution kernel that the calling
 * thread's last swc_winograd2x2_conv / _conv_bf16 / _conv_epilogue / _conv_bf16in / _conv_bf16in_ws call launched ("" before the
 * first): "sync" (any shape and alignment), "ring32" / "ring16" (64x64 tiles, 32- / 16-channel steps),
 * "tall16" / "short16" (row groups of up to 112 / 32 rows, dealt evenly over the CUs), "wide48" (48 rows x 128
 * columns per workgroup, left-over rows as extra tiles split along the channels; C % 64 == 0, K % 128 == 0),
 * "wide48x64" (the same with 64 columns per workgroup; K % 64 == 0); for
 * bf16-stored operands "stored-ring3" / "stored-ring4" (64x64 tiles, 3- / 4-deep copy ring) / "stored-split"
 * (small grids: the 16 positions of a tile split over two groups of waves, whose partial sums are added at the
 * end) / "stored-split4" (smaller grids still: 32-row tiles, four groups of waves) / "stored-tall" (128x64
 * tiles for C = 64, 128, 256 or 512 on grids that fill the device) / "stored-spread" (the same tiles, four workgroups
 * each, on grids far too small for it; swc_winograd2x2_conv_bf16in_ws with a scratch buffer only).  Which one runs
 * depends only on the shapes, pointer alignment, whether a scratch buffer was passed, and the device's CU count and
 * L2 size; all give the same results to within the order of the fp32 summations ("wide48", "stored-tall" and
 * "stored-spread" also add the nine terms of an output in another order than the rest: 1e-6 relative, exact on
 * integer-valued data). */
SWC_API const char *swc_winograd2x2_conv_last_kernel(void);
/* Diagnostic with no counterpart in the reference, for benchmarks and tests that compare the tilings: makes
 * the calling thread's later swc_winograd2x2_conv calls
 * use the named kernel ("ring32", "ring16", "tall16", "short16", "wide48", "wide48x64", "sync") where the shapes
 * allow it and "sync" where they do not; NULL or "" gives the choice back to the launcher.  The data gradient of
 * swc_winograd2x2_conv_grad follows it too: "wide48" takes its wide-tile kernel where the shapes allow it, any
 * other name its position-pair kernel.  Returns SWC_ERR_UNSUPPORTED for an unknown name. */
SWC_API int swc_winograd2x2_conv_force_tiling(const char *name);

/* ---------------------------------------------------------------------------
 * Launcher level: what the reference's TensorFlow op kernels call.
 * ------------------------------------------------------------------------- */

/*
 * Input transform T = B^T d B over 4x4 tiles at stride 2, pad 1, optionally followed by
 * the Winograd-domain ReLU.
 *   Input   [B,H,W,C]            fp32, NHWC, contiguous
 *   TransIm [16,B,nH,nW,C]       fp32, nH=(H+1)/2, nW=(W+1)/2
 * Replaces  void Winograd2x2ImTransComputeLauncher(const float *Input, float *TransIm,
 *           int C, int B, int H, int W, int pad_h, int pad_w)
 *   declared winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_op.cc:30,
 *   defined  winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_cuda.cu.cc:151-157,
 *   called   winograd2x2_imTrans_op.cc:55 (always with pad 1,1).
 * `relu` != 0 fuses the tf.nn.relu that the layer wrapper applies to the op's result
 * (ResNet-18-var/winograd_imtrans.py:16-17): t > 0 ? t : 0.  The 16 sums keep the
 * reference's left-to-right association (…_cuda.cu.cc:112-127), so values and zero
 * masks are bit-identical to it.  Unlike the reference, C is not limited to 1024.
 */
SWC_API int swc_winograd2x2_imtrans(const float *Input, float *TransIm, int C, int B, int H, int W,
                            int pad_h, int pad_w, int relu, swc_stream_t stream);

/*
 * swc_winograd2x2_imtrans with a per-channel affine map folded into the load: every pixel inside
 * the image becomes fmaf(x, Scale[c], Shift[c]) before the transform; the zero padding stays zero.
 *   Scale, Shift [C] fp32
 * This is the inference-mode BatchNorm that precedes every WinogradImTrans in the reference model
 * (`BatchNorm('bn2a_2a', x)` then `WinogradImTrans(..., tf.nn.relu)`,
 * ResNet-18-var/imagenet-resnet-transWino-prune.py:117-118 and the 15 other pairs up to :210), with
 * Scale = gamma / sqrt(var + eps), Shift = beta - mean * Scale: one pass over the activations
 * instead of two.  The reference has no single function for the pair.
 */
SWC_API int swc_winograd2x2_imtrans_affine(const float *Input, const float *Scale, const float *Shift,
                                   float *TransIm, int C, int B, int H, int W, int pad_h, int pad_w, int relu,
                                   swc_stream_t stream);

/*
 * The 16 per-position products TI[i] (MxC) . Weight[i] (CxK), M = B*nH*nW, followed by
 * the output transform Y = A^T p A, in one kernel (fp32 MFMA, fp32 accumulate).
 *   Input  [16,B,nH,nW,C]  fp32      Weight [16,C,K] fp32
 *   Output [B,2nH,2nW,K]   fp32, NHWC, never cropped
 * Replaces  void Winograd2x2ConvComputeLauncher(const float *Input, const float *Weight,
 *           float *Output, float *tmp_data_buffer, const long long *tmp_ptr_buffer,
 *           int C, int B, int nH, int nW, int K, int pad_h, int pad_w)
 *   declared winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_op.cc:31,
 *   defined  winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc:65-93
 *   (assign :55-61, cublasSgemmBatched :80-85, Output_transform :12-53,87-89),
 *   called   winograd2x2_conv_op.cc:66.
 * tmp_data_buffer (16*M*K floats there) and tmp_ptr_buffer (48 pointers there) are kept
 * in the signature for call-site compatibility and ignored: pass NULL.  The products
 * never leave registers.  Unlike the reference, K is not limited to 1024.
 */
SWC_API int swc_winograd2x2_conv(const float *Input, const float *Weight, float *Output,
                         float *tmp_data_buffer, const long long *tmp_ptr_buffer,
                         int C, int B, int nH, int nW, int K, int pad_h, int pad_w,
                         swc_stream_t stream);

/*
 * swc_winograd2x2_conv with per-element work folded into its output stores:
 *   Output = fmaf(conv, Scale[k], Shift[k]) + Residual        (residual_relu == 0)
 *   Output = fmaf(conv, Scale[k], Shift[k]) + max(Residual, 0) (residual_relu != 0: the identity shortcut of the
 *            units without a 1x1 conv is `relu(x)`, imagenet-resnet-transWino-prune.py:135-143)
 *   Scale, Shift [K] fp32 (both or neither); Residual [B,2nH,2nW,K] fp32; any of them may be NULL.
 *   precision: 0 = fp32 MFMA, 1 = bf16 operands (as swc_winograd2x2_conv_bf16).
 * No counterpart function in the reference: it is what follows its second convolution of every
 * residual unit -- `BatchNorm('bn2a_2c', x)` at inference and the `tf.add([x, bra])` with the shortcut
 * (ResNet-18-var/imagenet-resnet-transWino-prune.py:123,131 and the seven other units up to :213) --
 * applied while the result is still in registers instead of in two more passes over it.
 * Residual may alias Output (each element is read before it is written, by the same lane).
 */
SWC_API int swc_winograd2x2_conv_epilogue(const float *Input, const float *Weight, float *Output,
                                  const float *Scale, const float *Shift, const float *Residual, int residual_relu,
                                  int C, int B, int nH, int nW, int K, int pad_h, int pad_w,
                                  int precision, swc_stream_t stream);

/*
 * Same contract as swc_winograd2x2_conv, with both GEMM operands rounded to bf16
 * (round-to-nearest-even) on their way into the matrix cores; accumulation and the
 * output transform stay fp32.  No counterpart in the reference (its GEMM is cuBLAS
 * SGEMM, winograd2x2_conv_cuda.cu.cc:80-85); an opt-in speed/precision trade.
 */
SWC_API int swc_winograd2x2_conv_bf16(const float *Input, const float *Weight, float *Output,
                              float *tmp_data_buffer, const long long *tmp_ptr_buffer,
                              int C, int B, int nH, int nW, int K, int pad_h, int pad_w,
                              swc_stream_t stream);

/* ---------------------------------------------------------------------------
 * Op level: what the reference's OpKernel::Compute and shape functions do on the
 * host (read dims from the tensors, derive the output shape, call the launcher).
 * Shapes are int64 arrays in the reference's dimension order.
 * ------------------------------------------------------------------------- */

/*
 * Shape rule of Winograd2x2ImTrans: [B,H,W,C] -> [16,B,(H+1)/2,(W+1)/2,C].
 * winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans.py:20-27 and
 * winograd2x2_imTrans_op.cc:42-51.
 */
SWC_API int swc_winograd2x2_imtrans_op_shape(int in_rank, const int64_t *in_dims, int64_t out_dims[5]);

/*
 * Winograd2x2ImTransCudaOp::Compute (winograd2x2_imTrans_op.cc:36-56) with the output
 * passed in instead of allocated: validates that out_dims is what the shape rule gives,
 * then launches with pad 1,1.
 */
SWC_API int swc_winograd2x2_imtrans_op_compute(const float *input, int in_rank, const int64_t *in_dims,
                                       float *output, int out_rank, const int64_t *out_dims,
                                       int relu, swc_stream_t stream);

/*
 * Shape rule of Winograd2x2Conv: I [16,B,nH,nW,C], W [16,C,K] -> [B,2nH,2nW,K].
 * winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv.py:19-29 and
 * winograd2x2_conv_op.cc:45-53.  The reference checks ranks only; this also requires
 * I.dim0 == W.dim0 == 16 and W.dim1 == C.
 */
SWC_API int swc_winograd2x2_conv_op_shape(int in_rank, const int64_t *in_dims, int w_rank, const int64_t *w_dims,
                                  int64_t out_dims[4]);

/*
 * Winograd2x2ConvCudaOp::Compute (winograd2x2_conv_op.cc:37-67) with the output passed
 * in; no temporaries are needed.  precision: 0 = fp32 MFMA, 1 = bf16 operands.
 */
SWC_API int swc_winograd2x2_conv_op_compute(const float *input, int in_rank, const int64_t *in_dims,
                                    const float *weight, int w_rank, const int64_t *w_dims,
                                    float *output, int out_rank, const int64_t *out_dims,
                                    int precision, swc_stream_t stream);

/*
 * The layer pair in one kernel: swc_winograd2x2_imtrans(relu) followed by swc_winograd2x2_conv,
 * without the [16,B,nH,nW,C] intermediate ever reaching memory.
 *   Input [B,H,W,C], Weight [16,C,K]  ->  Output [B,2nH,2nW,K]   (fp32)
 * No single counterpart in the reference: it is the composition of its two launchers and the
 * tf.nn.relu between them, as the model applies them
 * (ResNet-18-var/imagenet-resnet-transWino-prune.py:118-119; winograd_imtrans.py:16-17;
 * winograd_conv.py:28).  The transformed activations are bit-identical to the stand-alone
 * transform's, and the products are folded in the same ascending order, so the result agrees with
 * the two-call sequence to GEMM rounding.
 * Needs C % 8 == 0, K % 4 == 0, Weight 16-byte and Input 8-byte aligned, and fewer than 2^30 input
 * elements; otherwise returns SWC_ERR_UNSUPPORTED and the caller uses the two entry points above
 * (which need the intermediate buffer this one has no room for).
 */
SWC_API int swc_winograd2x2_relu_conv(const float *Input, const float *Weight, float *Output,
                                      int C, int B, int H, int W, int K, int pad_h, int pad_w,
                                      int relu, swc_stream_t stream);

/* ---------------------------------------------------------------------------
 * bf16-stored variant of the forward pair (no counterpart in the reference, whose tensors are all
 * fp32): the transformed activations are written, kept and read as bf16, which halves the traffic of
 * the HBM-bound half of the path.  Arithmetic: the transform and its ReLU in fp32 exactly as in
 * swc_winograd2x2_imtrans, one rounding to bf16 (nearest even) on the store; the GEMMs multiply the
 * bf16 operands exactly and accumulate in fp32; output transform and output in fp32 -- the same
 * values swc_winograd2x2_conv_bf16 computes from the fp32 TransIm.
 * ------------------------------------------------------------------------- */

/* swc_winograd2x2_imtrans (Scale == Shift == NULL) or swc_winograd2x2_imtrans_affine, with
 * TransIm16 [16,B,nH,nW,C] stored as bf16 bit patterns. */
SWC_API int swc_winograd2x2_imtrans_bf16out(const float *Input, const float *Scale, const float *Shift,
                                    uint16_t *TransIm16, int C, int B, int H, int W, int pad_h, int pad_w,
                                    int relu, swc_stream_t stream);

/* Weight [16,C,K] fp32 -> Weight16t [16,K,C] bf16 (nearest even), the layout the kernel below reads.
 * Done once per weight update, like the W*mask of ResNet-18-var/winograd_conv.py:25. */
SWC_API int swc_winograd2x2_weights_bf16(const float *Weight, uint16_t *Weight16t, int C, int K, swc_stream_t stream);

/* swc_winograd2x2_conv_epilogue over the bf16 operands: Output [B,2nH,2nW,K] fp32 =
 * fmaf(conv, Scale[k], Shift[k]) + Residual (Scale/Shift/Residual may be NULL; residual_relu as above).  Needs C % 64 == 0 and
 * 16-byte aligned operands; returns SWC_ERR_UNSUPPORTED otherwise (use the fp32-stored path). */
SWC_API int swc_winograd2x2_conv_bf16in(const uint16_t *Input16, const uint16_t *Weight16t, float *Output,
                                const float *Scale, const float *Shift, const float *Residual, int residual_relu,
                                int C, int B, int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream);

/* swc_winograd2x2_conv_bf16in with a scratch buffer of the caller's (device memory, 16-byte aligned): what the
 * reference's tmp_data_buffer is to its launcher (winograd2x2_conv_op.cc:57-60 allocates 16*M*K floats per call,
 * winograd2x2_conv_cuda.cu.cc:65 takes them).  Layers of 256 or 512 channels with so few 128-row x 64-column tiles
 * that four times as many workgroups still find a CU each (7x7x512 at batch 64, 14x14x256 at batch 16) then run as
 * four workgroups per tile, one per row of the 4x4 position grid,
 * whose partial sums meet in the buffer; a second kernel combines them, applies the epilogue and writes the output.
 * swc_winograd2x2_conv_bf16in_workspace_floats says how many floats that takes on the current device (8*M*K, or 0
 * for shapes that do not use a buffer).  With Workspace NULL, or fewer than that many floats, the call is
 * swc_winograd2x2_conv_bf16in.  The sums of the output transform are then taken row by row of the position grid:
 * results agree with swc_winograd2x2_conv_bf16in to rounding, not bit for bit. */
SWC_API size_t swc_winograd2x2_conv_bf16in_workspace_floats(int C, int B, int nH, int nW, int K);
SWC_API int swc_winograd2x2_conv_bf16in_ws(const uint16_t *Input16, const uint16_t *Weight16t, float *Output,
                                   const float *Scale, const float *Shift, const float *Residual, int residual_relu,
                                   float *Workspace, size_t workspace_floats,
                                   int C, int B, int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream);

/* The whole layer in one kernel with bf16 GEMM operands: the values of swc_winograd2x2_imtrans_bf16out
 * (with InScale/InShift as in swc_winograd2x2_imtrans_affine, or NULL) followed by
 * swc_winograd2x2_conv_bf16in (with OutScale/OutShift/Residual as in swc_winograd2x2_conv_epilogue, or
 * NULL), without the transformed activations ever reaching memory.
 *   Input [B,H,W,C] fp32, Weight16t [16,K,C] bf16 (swc_winograd2x2_weights_bf16)  ->  Output [B,2nH,2nW,K] fp32
 * No counterpart in the reference.  Needs C % 16 == 0 and 16-byte aligned operands; returns
 * SWC_ERR_UNSUPPORTED otherwise (use the two entry points above). */
SWC_API int swc_winograd2x2_relu_conv_bf16(const float *Input, const float *InScale, const float *InShift,
                                   const uint16_t *Weight16t, float *Output, const float *OutScale,
                                   const float *OutShift, const float *Residual, int C, int B, int H, int W,
                                   int K, int pad_h, int pad_w, int relu, swc_stream_t stream);

/*
 * 1x1 convolution over NHWC pixels: Output [M,K] = Input [M,C] . Weight [K,C]^T, M = B*H*W, fp32.
 * No counterpart among the reference's custom ops: its model takes the shortcut of the first unit of every stage
 * through tensorpack's Conv2D (`Conv2D('res2a_1', l, 64, 1, ...)`, ResNet-18-var/imagenet-resnet-transWino-prune.py:127,
 * :152, :177, :202).  Here it runs on the kernel of the convolution's data gradient (one of its 16 products has
 * exactly this form), which reads and writes each byte once where the library GEMM PyTorch picks for these
 * skinny shapes takes 2-6 times as long.  Needs C % 32 == 0 and 16-byte aligned operands; returns
 * SWC_ERR_UNSUPPORTED otherwise (use any GEMM).
 */
SWC_API int swc_winograd2x2_pointwise_conv(const float *Input, const float *Weight, float *Output, int C, long long M,
                                           int K, swc_stream_t stream);

/* ---------------------------------------------------------------------------
 * Backward ops.
 * ------------------------------------------------------------------------- */

/*
 * Gradient of swc_winograd2x2_conv with respect to both inputs.
 *   TInput [16,B,nH,nW,C], Weight [16,C,K], Output_grad [B,H,W,K] with H = 2nH, W = 2nW
 *   -> TInput_grad [16,B,nH,nW,C], Weight_grad [16,C,K]
 * Replaces  void Winograd2x2ConvGradComputeLauncher(const float *TInput, const float *Weight,
 *           const float *Output_grad, float *TInput_grad, float *Weight_grad, float *tmp_data_buffer,
 *           long long *tmp_ptr_buffer, int C, int B, int H, int W, int K, int pad_h, int pad_w)
 *   declared winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_op.cc:32,
 *   defined  winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_cuda.cu.cc:77-124.
 * tmp_data_buffer must hold 16*B*nH*nW*K floats (the caller's temporary, as at
 * winograd2x2_conv_grad_op.cc:69-71); tmp_ptr_buffer is ignored.  TInput_grad is also used as
 * scratch (partial sums of Weight_grad) before it receives its result, so it must not alias an input.
 * Both GEMMs of the reference (:103-108, :115-120) run on this library's own kernels.
 */
SWC_API int swc_winograd2x2_conv_grad(const float *TInput, const float *Weight, const float *Output_grad,
                                      float *TInput_grad, float *Weight_grad, float *tmp_data_buffer,
                                      long long *tmp_ptr_buffer, int C, int B, int H, int W, int K,
                                      int pad_h, int pad_w, swc_stream_t stream);

/*
 * swc_winograd2x2_conv_grad for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc); it has no counterpart in the reference.  Same arguments and
 * results without the two temporaries: the 16*B*nH*nW*K floats of A dY A^T are kept in a fixed array in device
 * memory that the library holds on every GPU it runs on (SWC_CONV_GRAD_STATIC_MAX_FLOATS floats = 64 MiB, i.e.
 * B*nH*nW*K <= 1 048 576; larger calls return SWC_ERR_TOO_LARGE and launch nothing).  Nothing is allocated or
 * freed, by this call or by anything it calls.  All calls on one GPU share that array: calls that may overlap on
 * one GPU (different streams or host threads) race on it and must be serialised by the caller.
 * The first call on a device looks up the array's address there (hipGetDevice and hipGetSymbolAddress, under a
 * mutex): a caller that captures HIP graphs makes one call on the device outside the capture first.
 * The array is part of the library's code object, so every process that loads the library holds its 64 MiB on every
 * GPU it uses, whether or not it calls this entry point; a build for forward-only deployments can shrink it with
 * -DSWC_CONV_GRAD_STATIC_MAX_FLOATS=<n>.
 */
#ifndef SWC_CONV_GRAD_STATIC_MAX_FLOATS
#define SWC_CONV_GRAD_STATIC_MAX_FLOATS (16u << 20)
#endif
SWC_API int swc_winograd2x2_conv_grad_static(const float *TInput, const float *Weight, const float *Output_grad,
                                             float *TInput_grad, float *Weight_grad, int C, int B, int H, int W,
                                             int K, int pad_h, int pad_w, swc_stream_t stream);

/*
 * Gradient of swc_winograd2x2_imtrans: TransIm_grad [16,B,nH,nW,C] -> Input_grad [B,H,W,C].
 * Replaces  void Winograd2x2ImTransGradComputeLauncher(const float *Output_grad, float *Input_grad,
 *           int C, int B, int H, int W, int pad_h, int pad_w)
 *   declared winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_grad_op.cc:29,
 *   defined  winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_grad_cuda.cu.cc:118-129.
 * relu_mask_source, if not NULL, is the forward op's output computed with relu != 0: the gradient
 * is then taken through the fused ReLU (entries where it is <= 0 contribute nothing).  Unlike the
 * reference (:124), TransIm_grad is not overwritten.  H need not be even here (the reference's op
 * wrapper always passes H = 2nH, winograd2x2_imTrans_grad_op.cc:44-45).
 */
SWC_API int swc_winograd2x2_imtrans_grad(const float *TransIm_grad, const float *relu_mask_source,
                                         float *Input_grad, int C, int B, int H, int W,
                                         int pad_h, int pad_w, swc_stream_t stream);

/*
 * The same gradient through the fused ReLU, with the ReLU's mask recomputed from the forward
 * op's input instead of read from its output: Input [B,H,W,C] is what swc_winograd2x2_imtrans was
 * given (no scale/shift), and the transform's additions are repeated in the forward order, so the
 * mask is the forward pass's bit for bit.  Reads a quarter of the bytes the mask costs above and
 * lets a training caller keep [B,H,W,C] instead of [16,B,nH,nW,C] for this op's backward.
 * No counterpart in the reference, whose ReLU is a separate op (ResNet-18-var/winograd_imtrans.py:17).
 */
SWC_API int swc_winograd2x2_imtrans_grad_relu_input(const float *TransIm_grad, const float *Input,
                                                    float *Input_grad, int C, int B, int H, int W,
                                                    int pad_h, int pad_w, swc_stream_t stream);

/*
 * Shape rule of Winograd2x2ConvGrad: TInput [16,B,nH,nW,C], Weight [16,C,K], Output_grad [B,H,W,K] with
 * H = 2nH, W = 2nW -> the two results shaped like TInput and Weight, and the number of floats of the temporary
 * the launcher needs (16*nH*nW*B*K), as Winograd2x2ConvGradCudaOp::Compute derives them
 * (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_op.cc:44-67).  The reference checks nothing; this
 * also requires that the three shapes agree.
 */
SWC_API int swc_winograd2x2_conv_grad_op_shape(int ti_rank, const int64_t *ti_dims, int w_rank, const int64_t *w_dims,
                                       int g_rank, const int64_t *g_dims, int64_t ti_grad_dims[5],
                                       int64_t w_grad_dims[3], int64_t *tmp_floats);

/*
 * Winograd2x2ConvGradCudaOp::Compute (winograd2x2_conv_grad_op.cc:36-78) with the two results and the temporary
 * passed in (tmp_floats: how many floats tmp_data_buffer holds); launches with pad 1,1.
 */
SWC_API int swc_winograd2x2_conv_grad_op_compute(const float *tinput, int ti_rank, const int64_t *ti_dims,
                                         const float *weight, int w_rank, const int64_t *w_dims,
                                         const float *output_grad, int g_rank, const int64_t *g_dims,
                                         float *tinput_grad, float *weight_grad, float *tmp_data_buffer,
                                         int64_t tmp_floats, swc_stream_t stream);

/*
 * Shape rule of Winograd2x2ImTransGrad: Output_grad [16,B,nH,nW,C] -> [B,2nH,2nW,C]
 * (winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_grad_op.cc:40-49).
 */
SWC_API int swc_winograd2x2_imtrans_grad_op_shape(int g_rank, const int64_t *g_dims, int64_t in_grad_dims[4]);

/*
 * Winograd2x2ImTransGradCudaOp::Compute (winograd2x2_imTrans_grad_op.cc:33-55) with the result passed in.
 * ig_dims is [B,H,W,C] with H = 2nH as in the reference, or 2nH - 1 for a forward input of odd extent (likewise
 * W).  relu_output / relu_input: at most one of them, the source of the fused ReLU's mask as in
 * swc_winograd2x2_imtrans_grad / swc_winograd2x2_imtrans_grad_relu_input; both NULL: no ReLU, as in the reference.
 */
SWC_API int swc_winograd2x2_imtrans_grad_op_compute(const float *output_grad, int g_rank, const int64_t *g_dims,
                                            const float *relu_output, const float *relu_input,
                                            float *input_grad, int ig_rank, const int64_t *ig_dims,
                                            swc_stream_t stream);

#ifdef __cplusplus
} /* extern "C" */

/*
 * C++ linkage, exact reference signatures: an unmodified winograd2x2_imTrans_op.cc /
 * winograd2x2_conv_op.cc (which declare these at :30 / :31 and call them at :55 / :66)
 * links against this library in place of the CUDA objects.  They run on the null
 * stream, as the reference launches do, apply no ReLU, and report errors on stderr
 * because the signatures return void.
 */
SWC_API void Winograd2x2ImTransComputeLauncher(const float *Input, float *TransIm, int C, int B, int H, int W,
                                       int pad_h, int pad_w);
SWC_API void Winograd2x2ConvComputeLauncher(const float *Input, const float *Weight, float *Output,
                                    float *tmp_data_buffer, const long long *tmp_ptr_buffer,
                                    int C, int B, int nH, int nW, int K, int pad_h, int pad_w);
/* Likewise for the gradient ops (winograd2x2_conv_grad_op.cc:32,77; winograd2x2_imTrans_grad_op.cc:29,54). */
SWC_API void Winograd2x2ConvGradComputeLauncher(const float *TInput, const float *Weight, const float *Output_grad,
                                        float *TInput_grad, float *Weight_grad, float *tmp_data_buffer,
                                        long long *tmp_ptr_buffer, int C, int B, int H, int W, int K,
                                        int pad_h, int pad_w);
SWC_API void Winograd2x2ImTransGradComputeLauncher(const float *Output_grad, float *Input_grad, int C, int B,
                                           int H, int W, int pad_h, int pad_w);
#endif

#endif /* WINOGRAD2X2_H_ */
