/*
 * ogle_hip.h - C ABI of the MI355X (gfx950) kernels behind OGLE's convolution
 * hot path.
 *
 * This is the boundary the reference's "Program" layer is replaced at.  In the
 * reference, Kernel::Compute sets uniforms on a GLSL program and issues one
 * draw call (ogl_runtime/opengl/core/program.h:30-103, used by
 * ogl_runtime/opengl/nn/kernels/conv2d.cc:116-167).  Here the same call sites
 * fill a plain struct and call one entry point, which launches hand-written
 * HIP kernels on the given stream.
 *
 * Conventions
 *  - Every pointer named *_dev is device memory owned by the caller.  Unless an
 *    entry point says otherwise nothing here allocates, frees or synchronises:
 *    launches are asynchronous on `stream`.
 *  - Activations are dense NHWC, channel contiguous, no per-pixel padding.
 *    Logical shapes are the reference's (Tensor::shape() NHWC, filters OIHW).
 *  - Filters are consumed in a packed device layout produced once at load time
 *    by ogle_hip_pack_filter (the counterpart of the reference's
 *    NCHW -> HWN4C4 upload, ogl_runtime/opengl/nn/kernels/const.cc:21-28).
 *  - Return value: OGLE_OK (0) or a negative OgleStatus.  Entry points never
 *    abort; ogle_hip_last_error() gives the message of the calling thread's
 *    last failure.  The reference aborts through glog CHECK / LOG(FATAL)
 *    (ogl_runtime/opengl/utils/macros.h:16-20); its Kernel wrappers turn a
 *    non-zero status back into that behaviour.
 *  - `stream` is a hipStream_t passed as void* so that this header needs no
 *    HIP include; NULL is the default stream.
 */
#ifndef OGLE_HIP_H_
#define OGLE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ogle_stream_t;

typedef enum OgleStatus {
  OGLE_OK = 0,
  OGLE_ERR_INVALID_ARG = -1, /* shape/attribute violates what the op allows */
  OGLE_ERR_UNSUPPORTED = -2, /* valid request, no kernel for it             */
  OGLE_ERR_LAUNCH = -3,      /* HIP reported an error at launch             */
  OGLE_ERR_NOT_FOUND = -4,   /* registry lookup failed                      */
  OGLE_ERR_NO_DEVICE = -5    /* no gfx950 device / code object              */
} OgleStatus;

typedef enum OgleDType { OGLE_F32 = 0, OGLE_F16 = 1 } OgleDType;

/* Fused activation codes: the reference's "act" uniform
 * (ogl_runtime/opengl/nn/kernels/conv2d.cc:137-147). */
typedef enum OgleAct { OGLE_ACT_NONE = 0, OGLE_ACT_CLIP = 1, OGLE_ACT_RELU = 2 } OgleAct;

/* How a shader variant reads min/max for the fused activation.
 * NHWC4: conv2d.glsl:82-90 (clamp(x,min,max); relu max(0,x)).
 * PW:    conv2d_pw.glsl:85 (clamp(x,0,max): min ignored).
 * ANY4:  conv2d_any4.glsl:89-94, conv2d_dw_any4.glsl:90-97, conv2d_pw_any4.glsl:80-87
 *        and conv2d_grp.glsl:115-121 (clip (min,max); relu is max(min,x)). */
typedef enum OgleActVariant {
  OGLE_VARIANT_NHWC4 = 0,
  OGLE_VARIANT_PW = 1,
  OGLE_VARIANT_ANY4 = 2
} OgleActVariant;

/* Packed filter layouts. */
typedef enum OgleFilterLayout {
  OGLE_FILTER_OHWI = 0, /* [O][kh][kw][I/g]: dense, pointwise, grouped */
  OGLE_FILTER_HWC = 1   /* [kh*kw][C]: depthwise (multiplier 1)        */
} OgleFilterLayout;

/* ------------------------------------------------------------------------ */
/* Library / registry                                                         */
/* ------------------------------------------------------------------------ */

/* Version of this ABI (major*100 + minor). */
int32_t ogle_hip_abi_version(void);

/* Number of device operations (kernels, and the one device-to-device copy an identity
 * transpose makes) the calling thread has enqueued through this library so far.  The
 * difference across a call says how many dispatches that call became, which is how a
 * profiler trace of a replayed pass is lined up with the graph's nodes. */
int64_t ogle_hip_launch_count(void);

/*
 * Kernel timing.  Between _begin and _end every kernel the calling thread launches through
 * this library carries its own start / stop HIP events, stamped by the device with the
 * kernel's own begin and end (no launch gaps, unlike events recorded between launches), so
 * the durations are the ones a profiler's kernel trace shows.  _end waits for the kernels,
 * writes their durations in launch order (one entry per device operation counted by
 * ogle_hip_launch_count; 0 for an operation that is not a kernel) and returns how many
 * there were (may exceed `capacity`), or a negative status.  Not for use while the stream
 * is being captured.  The reference's counterpart is its per-node TraceMe scope with
 * glFinish (ogl_runtime/opengl/core/fbo_session.cc:128-151).
 */
int32_t ogle_hip_kernel_timing_begin(void);
int64_t ogle_hip_kernel_timing_end(float* microseconds, int64_t capacity);

/* Message of the calling thread's most recent failure ("" if none). */
const char* ogle_hip_last_error(void);
const char* ogle_hip_status_string(int32_t status);

/*
 * Kernel registry: replaces the generated shader table (all_shaders.h, built
 * by ogl_runtime/opengl/nn/makeshader.py:16-43) and the program cache of
 * Context::CreateProgram (ogl_runtime/opengl/core/context.cc:288-313).
 * `name` is the shader's stem ("conv2d", "conv2d_dw", "conv2d_pw",
 * "conv2d_grp", "conv2d_any4", "conv2d_dw_any4", "conv2d_pw_any4", "pool",
 * "pool_any4", "concat_multi", "decoder"); `options` is the build-option text
 * the Kernel composed ("#define USE_BIAS\n#define USE_CLIP\n", may be NULL).
 * On success *handle identifies the HIP kernel family and its compile-time
 * flags; it is what OgleConvArgs.kernel carries.
 */
int32_t ogle_hip_registry_lookup(const char* name, const char* options, int32_t* handle);
int32_t ogle_hip_registry_size(void);
const char* ogle_hip_registry_name(int32_t index);

/* Waits for everything queued on `stream` (glFinish's counterpart,
 * ogl_runtime/opengl/nn/profiler/traceme.h:61-65). */
int32_t ogle_hip_sync(ogle_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Filter upload                                                              */
/* ------------------------------------------------------------------------ */

/* Number of elements of the packed filter for an OIHW filter (o, i, kh, kw). */
int64_t ogle_hip_packed_filter_elems(int32_t layout, int32_t o, int32_t i, int32_t kh,
                                     int32_t kw);

/*
 * Repacks an OIHW fp32 filter (device memory, the order the .dlx file stores,
 * converter/converter/onnx/ops/conv2d.cc:12-27) into `layout` with element type
 * `dtype`.  Counterpart of functor::ConvertTensorNCHWToHWN4C4
 * (ogl_runtime/opengl/core/functor.cc:45-93, shader nchw_to_hwn4c4.glsl).
 * For OGLE_FILTER_HWC, i must be 1.
 */
int32_t ogle_hip_pack_filter(const float* oihw_dev, void* packed_dev, int32_t layout,
                             int32_t dtype, int32_t o, int32_t i, int32_t kh, int32_t kw,
                             ogle_stream_t stream);

/* Element-type conversion of a flat buffer (fp32 <-> fp16 storage). */
int32_t ogle_hip_convert(const void* src_dev, int32_t src_dtype, void* dst_dev,
                         int32_t dst_dtype, int64_t count, ogle_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Convolution                                                                */
/* ------------------------------------------------------------------------ */

/*
 * Arguments of one convolution launch: the uniforms and texture bindings of
 * Conv2DKernel::Compute (ogl_runtime/opengl/nn/kernels/conv2d.cc:127-164).
 */
typedef struct OgleConvArgs {
  const void* input_dev;  /* NHWC (n, in_h, in_w, in_c), dtype               */
  const void* filter_dev; /* packed by ogle_hip_pack_filter, dtype            */
  const float* bias_dev;  /* (out_c) fp32, or NULL (no USE_BIAS)              */
  void* output_dev;       /* NHWC (n, out_h, out_w, out_c), dtype             */
  int32_t n, in_h, in_w, in_c;
  int32_t out_h, out_w, out_c;
  int32_t kernel_size, stride, padding, dilation, group;
  int32_t act;         /* OgleAct                                             */
  float min_value;     /* "min_value" uniform                                 */
  float max_value;     /* "max_value" uniform                                 */
  int32_t act_variant; /* OgleActVariant                                      */
  int32_t dtype;       /* OgleDType of input/filter/output; accumulation fp32 */
  /* Optional scratch for kernels that split the contraction over workgroups (few
   * output tiles, long K).  NULL / 0 is always valid: the launch then uses a plan
   * that needs none.  Launches on one stream may share one workspace. */
  void* workspace_dev;
  size_t workspace_bytes;
  /* Optional second destination (NULL: none).  With output2_dev set, 0 < out_c_split <
   * out_c and the convolution's output channels are divided between two dense NHWC
   * tensors: channels [0, out_c_split) of every pixel go to output_dev (out_c_split
   * channels per pixel), channels [out_c_split, out_c) to output2_dev (out_c -
   * out_c_split channels per pixel).  filter_dev and bias_dev cover all out_c channels.
   * This is how two convolutions that read the same input with the same geometry (the
   * box and class head of one SSD feature map) run as ONE contraction that fetches the
   * input once; the reference draws them one after the other (fbo_session.cc:140-153).
   * Only the MFMA implicit-GEMM path takes it (group 1, in_c % 4 == 0, k*k*in_c >= 32;
   * fp16 storage: in_c % 8 == 0): otherwise OGLE_ERR_UNSUPPORTED. */
  void* output2_dev;
  int32_t out_c_split;
  /* Optional distance, in elements, between the first outputs of consecutive images in
   * output_dev (0: the images follow each other, out_h * out_w * out_c apart).  A larger
   * value leaves a gap after every image: each image's out_h * out_w * out_c outputs stay
   * contiguous, and image b starts at output_dev + b * out_image_stride.  This is how a
   * convolution writes straight into its place inside the output of a Concat over axis 1
   * (the SSD box and class heads at batch > 1), which then has nothing left to copy; the
   * reference draws the head, then copies it (concat.cc:49-99).  Must be 0 or at least
   * out_h * out_w * out_c, and cannot be combined with output2_dev.  Only the MFMA
   * implicit-GEMM path takes it (ogle_hip_conv_takes_image_stride): otherwise
   * OGLE_ERR_UNSUPPORTED. */
  int64_t out_image_stride;
} OgleConvArgs;

/* 1 if a convolution of this geometry and dtype runs on a path that honours
 * out_image_stride, 0 if not (pointers are not looked at). */
int32_t ogle_hip_conv_takes_image_stride(const OgleConvArgs* args);

/* Bytes of workspace the fastest plan for `args` would use (0 if it needs none). */
size_t ogle_hip_conv_workspace_bytes(const OgleConvArgs* args);

/* Dense (group 1) or grouped KxK convolution: conv2d.glsl:29-92,
 * conv2d_grp.glsl:30-123, conv2d_any4.glsl:29-96.  Filter layout OHWI. */
int32_t ogle_hip_conv2d(const OgleConvArgs* args, ogle_stream_t stream);

/*
 * `count` mutually independent dense / pointwise convolutions (group 1) in as few
 * launches as possible: the result of each equals ogle_hip_conv2d on it alone, but
 * problems that use the same MFMA kernel share one grid, so several small
 * convolutions (the SSD heads) fill the chip side by side instead of one after the
 * other.  No convolution may read or write another's output, and workspaces must
 * not be shared between them.  The reference has no counterpart (it draws one node
 * at a time, fbo_session.cc:140-153); the runtime batches consecutive independent
 * Conv nodes into this call.
 */
int32_t ogle_hip_conv2d_batch(const OgleConvArgs* args, int32_t count, ogle_stream_t stream);

/*
 * ogle_hip_conv2d_batch in two steps, for convolutions whose results are not needed at
 * once (the SSD heads, read only by the final concat).  _begin launches the contractions
 * like ogle_hip_conv2d_batch but leaves the reductions of split-K plans unlaunched:
 * reduce_pending[i] is set to 1 for every convolution whose partial sums still sit in its
 * workspace (its output is not valid yet), 0 for the finished ones.  _finish, given those
 * same arguments (any subset, any order, from one or several _begin calls on the stream),
 * launches all their reductions as one grid per 16 convolutions.  The workspaces must stay
 * untouched in between.  One reduction grid at the end of a pass replaces one small
 * dependent launch per convolution.
 */
int32_t ogle_hip_conv2d_batch_begin(const OgleConvArgs* args, int32_t count,
                                    int32_t* reduce_pending, ogle_stream_t stream);
int32_t ogle_hip_conv2d_batch_finish(const OgleConvArgs* args, int32_t count, ogle_stream_t stream);

/*
 * ogle_hip_conv2d for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same kernels, same plans and bit-identical results
 * as ogle_hip_conv2d called with the workspace ogle_hip_conv_workspace_bytes asks
 * for, but the split-K partial sums go to a fixed array of
 * OGLE_CONV_NOALLOC_SCRATCH_BYTES inside the library's device image (every GPU the
 * library runs on holds it until the process ends) instead of a caller buffer.
 *  - args->workspace_dev must be NULL and workspace_bytes 0.
 *  - A convolution whose split-K plan needs more than the array holds is refused
 *    with OGLE_ERR_INVALID_ARG and a message naming both sizes; nothing is launched.
 *  - The call allocates and frees nothing and does not synchronise.  The array's
 *    address is looked up at the first call on each device (a symbol lookup, not an
 *    allocation); make that first call outside a stream capture.
 *  - All calls on one GPU share the one array: calls that may overlap in time on one
 *    GPU (different streams, different threads) race.  Calls on one stream are safe.
 */
#define OGLE_CONV_NOALLOC_SCRATCH_BYTES (16u << 20)
int32_t ogle_hip_conv2d_noalloc(const OgleConvArgs* args, ogle_stream_t stream);

/* Depthwise KxK (group == in_c == out_c): conv2d_dw.glsl:38-96,
 * conv2d_dw_any4.glsl:38-98.  Filter layout HWC. */
int32_t ogle_hip_dwconv2d(const OgleConvArgs* args, ogle_stream_t stream);

/* Pointwise 1x1, stride 1, pad 0, group 1, as a GEMM
 * [n*h*w, in_c] x [out_c, in_c]^T: conv2d_pw.glsl:35-91,
 * conv2d_pw_any4.glsl:35-88.  Filter layout OHWI (== [O][I]). */
int32_t ogle_hip_pwconv_gemm(const OgleConvArgs* args, ogle_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Pooling                                                                    */
/* ------------------------------------------------------------------------ */

/* pool_type as ogl_runtime/opengl/nn/kernels/pool.h:10-14. */
typedef enum OglePoolType { OGLE_POOL_MAX = 0, OGLE_POOL_AVG = 1, OGLE_POOL_GLOBAL_AVG = 2 } OglePoolType;

/* Uniforms of PoolKernel::Compute (ogl_runtime/opengl/nn/kernels/pool.cc:53-79). */
typedef struct OglePoolArgs {
  const void* input_dev; /* NHWC */
  void* output_dev;      /* NHWC (n, out_h, out_w, c) */
  int32_t n, in_h, in_w, c;
  int32_t out_h, out_w;
  int32_t kernel_size, stride, padding;
  int32_t pool_type; /* OglePoolType; for GLOBAL_AVG the caller sets
                        kernel_size = in_h, stride 1, padding 0 (pool.cc:84-91) */
  int32_t dtype;
} OglePoolArgs;

/* pool.glsl:19-66 / pool_any4.glsl. */
int32_t ogle_hip_pool2d(const OglePoolArgs* args, ogle_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Concat                                                                     */
/* ------------------------------------------------------------------------ */

#define OGLE_CONCAT_MAX_INPUTS 16

/*
 * Concatenation of n_inputs tensors along one axis: ConcatKernel::Compute
 * (ogl_runtime/opengl/nn/kernels/concat.cc:56-97) with the intended semantics
 * of concat_multi.glsl:14-114 (numpy.concatenate).  Each input i is viewed as
 * (outer, axis_len[i], inner) row-major and lands at its running offset along
 * the axis of the (outer, sum axis_len, inner) output.  One launch for all
 * inputs.  n_inputs <= OGLE_CONCAT_MAX_INPUTS.  With outer == 1 the output is the
 * inputs back to back: if every input already lies at its place inside the output
 * (the runtime lets the producers write there), nothing is launched; an input may
 * not overlap the output in any other way.
 */
typedef struct OgleConcatArgs {
  const void* inputs_dev[OGLE_CONCAT_MAX_INPUTS];
  int64_t axis_len[OGLE_CONCAT_MAX_INPUTS];
  void* output_dev;
  int32_t n_inputs;
  int64_t outer;
  int64_t inner;
  int32_t dtype;
} OgleConcatArgs;

int32_t ogle_hip_concat(const OgleConcatArgs* args, ogle_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Transpose                                                                  */
/* ------------------------------------------------------------------------ */

/*
 * Permutation of a rank-4 row-major tensor: output dimension d is input
 * dimension perm[d] (out_shape[d] == in_shape[perm[d]]).  Uniforms of
 * TransposeKernel::Compute (ogl_runtime/opengl/nn/kernels/transpose.cc:71-89,
 * shaders transpose.glsl / transpose_any4.glsl); lower ranks are left-padded with
 * 1s by the caller as AmendShape / AmendPerm do (transpose.cc:13-31).
 */
typedef struct OgleTransposeArgs {
  const void* input_dev;
  void* output_dev;
  int32_t in_shape[4];
  int32_t perm[4];
  int32_t dtype;
} OgleTransposeArgs;

int32_t ogle_hip_transpose(const OgleTransposeArgs* args, ogle_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Elementwise ops and Gemm (classification graphs)                           */
/* ------------------------------------------------------------------------ */

typedef enum OgleUnaryOp {
  OGLE_UNARY_RELU = 0, /* relu.glsl:8-10: max(0, x) */
  OGLE_UNARY_CLIP = 1  /* clip.glsl:7-12: min(max_value, max(min_value, x)) */
} OgleUnaryOp;

/* ReluKernel / ClipKernel (ogl_runtime/opengl/nn/kernels/{relu,clip}.cc).  `count`
 * elements of any shape; input and output may be the same buffer.  Pointers must
 * be 16-byte aligned. */
typedef struct OgleUnaryArgs {
  const void* input_dev;
  void* output_dev;
  int64_t count;
  int32_t op; /* OgleUnaryOp */
  float min_value, max_value;
  int32_t dtype;
} OgleUnaryArgs;

int32_t ogle_hip_unary(const OgleUnaryArgs* args, ogle_stream_t stream);

/* BinaryKernel, registered as "Add" (ogl_runtime/opengl/nn/kernels/binary.cc,
 * binary.glsl:8): y = a + b over two tensors of one shape. */
typedef struct OgleBinaryArgs {
  const void* a_dev;
  const void* b_dev;
  void* output_dev;
  int64_t count;
  int32_t dtype;
} OgleBinaryArgs;

int32_t ogle_hip_add(const OgleBinaryArgs* args, ogle_stream_t stream);

/* BatchNormKernel (ogl_runtime/opengl/nn/kernels/batchnorm.cc, batchnorm.glsl:33):
 * y = (x - mean) / sqrt(var + eps) * gamma + beta, the four fp32 parameter vectors
 * indexed by the last dimension (`channels`); `outer` is the product of the others. */
typedef struct OgleBatchNormArgs {
  const void* input_dev;
  const float* gamma_dev;
  const float* beta_dev;
  const float* mean_dev;
  const float* var_dev;
  void* output_dev;
  int64_t outer;
  int32_t channels;
  float epsilon;
  int32_t dtype;
} OgleBatchNormArgs;

int32_t ogle_hip_batchnorm(const OgleBatchNormArgs* args, ogle_stream_t stream);

/* GemmKernel (ogl_runtime/opengl/nn/kernels/gemm.cc, gemm.glsl:33-95), fp32:
 * Y(M,N) = alpha * A(M,K) * B' + beta * C, where B' is B(K,N) or, with trans_b, the
 * transpose of B(N,K).  C is NULL, a row of N values added to every row of Y
 * (c_rank 1), or (M,N) (c_rank 2) as in GemmCPU (gemm_test.cc:9-40).  The Linear
 * form (trans_b, alpha 1, C NULL or a row with beta 1, K % 4 == 0) runs on the MFMA
 * units and may use a workspace of ogle_hip_gemm_workspace_bytes() bytes for its
 * split-K plans (optional; the library does not allocate). */
typedef struct OgleGemmArgs {
  const float* a_dev;
  const float* b_dev;
  const float* c_dev;
  float* y_dev;
  int32_t m, n, k;
  int32_t trans_b;
  int32_t c_rank;
  float alpha, beta;
  void* workspace_dev;
  size_t workspace_bytes;
} OgleGemmArgs;

size_t ogle_hip_gemm_workspace_bytes(const OgleGemmArgs* args);
int32_t ogle_hip_gemm(const OgleGemmArgs* args, ogle_stream_t stream);

/* ------------------------------------------------------------------------ */
/* SSD box decoder and score filter                                           */
/* ------------------------------------------------------------------------ */

/*
 * Box decode: decoder.glsl:13-28 as driven by DecoderKernel::Compute
 * (ogl_runtime/opengl/nn/kernels/decoder.cc:33-58) and
 * functor::SSDBBoxDecoder (ogl_runtime/opengl/core/functor.cc:96-143).
 * prediction (batch, priors, 4) = (tx,ty,tw,th); anchors (cx,cy,w,h);
 * output (batch, priors, 4) = (xmin,ymin,xmax,ymax).  anchors_batch_stride is
 * 0 when every image shares one (priors,4) anchor set (the functor form) or
 * priors*4 when anchors are (batch, priors, 4) (the graph-op form,
 * decoder.cc:82-85).
 */
typedef struct OgleDecodeArgs {
  const float* prediction_dev;
  const float* anchors_dev;
  float* boxes_dev;
  int32_t batch, priors;
  int64_t anchors_batch_stride;
  float variances[4];
} OgleDecodeArgs;

int32_t ogle_hip_ssd_decode(const OgleDecodeArgs* args, ogle_stream_t stream);

/*
 * Decode + per-prior softmax-max + score threshold + ordered compaction, in
 * one launch: decoder.glsl followed by Detector::GenerateBoxInfo
 * (ogl_runtime/opengl/examples/ssd/detector.cc:184-225), for every image of
 * the batch.  Outputs per image b, in ascending prior order:
 *   kept_count_dev[b]
 *   kept_prior_dev[b*priors + r], kept_class_dev[..], kept_score_dev[..]
 *   kept_box_dev[(b*priors + r)*4 + 0..3]  scaled xmin,ymin,xmax,ymax (fp32)
 *   kept_rect_dev[(b*priors + r)*4 + 0..3] integer x,y,width,height
 *                                          (cv::Rect truncation, detector.cc:211-214)
 * boxes_dev (batch, priors, 4), if not NULL, also receives every decoded box
 * (what the reference reads back).  If prediction_dev is NULL, boxes_dev is an
 * INPUT holding already decoded boxes.  Any kept_* pointer except
 * kept_count_dev may be NULL.
 *
 * kept_count_dev == NULL asks for the lists IN PLACE instead: no compaction pass,
 * every prior's record stays at its own slot [b*priors + i] and kept_prior_dev holds
 * i for a kept prior and -1 for a dropped one (the other lists are written for every
 * prior).  All five lists are then required.  ogle_hip_ssd_topk_nms takes such lists
 * when its kept_count_dev is NULL; a caller that only wants the final detections
 * saves one launch per pass this way.
 */
typedef struct OgleDetectArgs {
  const float* logits_dev;     /* (batch, priors, classes) */
  const float* prediction_dev; /* (batch, priors, 4) or NULL */
  const float* anchors_dev;    /* as OgleDecodeArgs */
  float* boxes_dev;            /* (batch, priors, 4), see above */
  int32_t batch, priors, classes;
  int64_t anchors_batch_stride;
  float variances[4];
  float score_threshold; /* strict > (detector.cc:209) */
  float image_width;     /* scale applied to x (detector.cc:201-204) */
  float image_height;
  int32_t* kept_count_dev;
  int32_t* kept_prior_dev;
  int32_t* kept_class_dev;
  float* kept_score_dev;
  float* kept_box_dev;
  int32_t* kept_rect_dev;
} OgleDetectArgs;

int32_t ogle_hip_ssd_detect(const OgleDetectArgs* args, ogle_stream_t stream);

/*
 * Top-k by score, then NMS, per image, on the lists ogle_hip_ssd_detect leaves
 * on the device: Detector::GetTopK + Detector::NMS
 * (ogl_runtime/opengl/examples/ssd/detector.cc:114-148) with iou() of
 * examples/ssd/common.cc:57-77 on the integer rectangles.
 *   - order: score descending; entries with equal scores keep their order in the
 *     kept list (ascending prior index).  The reference's std::sort leaves the
 *     order of equal scores unspecified; this is the stable choice.
 *   - the first min(count, topk) entries go to NMS: entry j is dropped if any
 *     earlier entry i has iou(i, j) > nms_threshold (strict), whether or not i
 *     was itself dropped (detector.cc:130-141).
 * kept_count_dev == NULL: the lists are in place as ogle_hip_ssd_detect leaves them
 * without kept_count_dev (all `stride` slots are looked at, kept_prior_dev < 0 marks
 * an empty one); the results are the same.
 * Inputs are indexed [b*stride + r], r < kept_count_dev[b]; outputs
 * [b*topk + r], r < final_count_dev[b], in sorted order.  kept_box_dev /
 * final_box_dev may both be NULL.  1 <= topk <= 1024, stride <= 8192 and
 * 4*stride + 28*topk + 1.2 KB must fit 64 KB of LDS (OGLE_ERR_UNSUPPORTED otherwise).
 */
typedef struct OgleNmsArgs {
  const int32_t* kept_count_dev;
  const int32_t* kept_prior_dev;
  const int32_t* kept_class_dev;
  const float* kept_score_dev;
  const float* kept_box_dev;
  const int32_t* kept_rect_dev;
  int32_t batch;
  int32_t stride; /* entries per image in the kept_* arrays (= priors) */
  int32_t topk;
  float nms_threshold;
  int32_t* final_count_dev;
  int32_t* final_prior_dev;
  int32_t* final_class_dev;
  float* final_score_dev;
  float* final_box_dev;
  int32_t* final_rect_dev;
} OgleNmsArgs;

int32_t ogle_hip_ssd_topk_nms(const OgleNmsArgs* args, ogle_stream_t stream);

/* y[i] = exp(x[i]) exactly as ogle_hip_ssd_detect evaluates it; lets a test
 * compare the device exponential with the host's on the same inputs. */
int32_t ogle_hip_expf(const float* x_dev, float* y_dev, int64_t count, ogle_stream_t stream);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* OGLE_HIP_H_ */
