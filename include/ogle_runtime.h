/*
 * ogle_runtime.h - C ABI of the graph runtime (libogle_runtime.so).
 *
 * The runtime itself is C++ and keeps the reference's classes (opengl::Kernel,
 * KernelRegistry, FBOSession, Tensor, Context, Detector; headers under
 * ogle_amd/runtime/opengl).  These entry points expose FBOSession's public
 * interface (ogl_runtime/opengl/core/fbo_session.h:20-51) and the SSD Detector
 * (ogl_runtime/opengl/examples/ssd/detector.h:28-79) to callers that cannot link
 * C++: tests and benchmarks drive the executor through them from Python.
 *
 * A fatal condition (the reference's CHECK / LOG(FATAL) abort) surfaces here as a
 * negative return value; ogle_rt_last_error() holds its "file:line message".
 */
#ifndef OGLE_RUNTIME_H_
#define OGLE_RUNTIME_H_

#include <stddef.h>
#include <stdint.h>

#include "ogle_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct OgleSession OgleSession; /* an opengl::FBOSession plus its Context */

const char* ogle_rt_last_error(void);

/* FBOSession(): one context (one HIP stream) per session. */
OgleSession* ogle_rt_session_create(void);
void ogle_rt_session_destroy(OgleSession* s);

/* FBOSession::LoadGraph(path) / LoadGraph(ModelProto) from serialized bytes
 * (fbo_session.cc:62-124). */
int32_t ogle_rt_load_file(OgleSession* s, const char* path);
int32_t ogle_rt_load_bytes(OgleSession* s, const void* data, size_t size);

/*
 * FBOSession::Run(NamedTensorList) (fbo_session.cc:127-165).  Input i is a host
 * float buffer named names[i] of LOGICAL shape dims[i][0..ranks[i]) whose element order
 * is dformats[i]: "NHWC", "NCHW" or "ANY" (dense, the product of the dims), or one of
 * the reference's stride-4 layouts "NHWC4", "ANY4", "HWN4C4"
 * (tensor_format.cc:272-343), whose buffers are larger than the product of the dims.
 * The buffer must hold ogle_rt_host_elements(dims[i], ranks[i], dformats[i]) floats:
 * that many are read.  The first call allocates every tensor.
 */
int32_t ogle_rt_run(OgleSession* s, int32_t n_inputs, const char* const* names,
                    const float* const* data, const int32_t* const* dims, const int32_t* ranks,
                    const char* const* dformats);

/*
 * Floats a host buffer of logical shape dims[0..rank) holds in layout `dformat`
 * (CalcAllocatedSize1D/2D, tensor_format.cc:251-343): the product of the dims for
 * "NHWC" / "NCHW" / "ANY"; n*h*w*4*ceil(c/4) for "NHWC4"; the last dim rounded up to 4
 * for "ANY4"; kh*kw*ceil(o/4) rows of 4*ceil(i/4) texels of 4 for "HWN4C4" (dims OIHW).
 * Negative status for an unknown tag or a rank the layout does not take.
 */
int64_t ogle_rt_host_elements(const int32_t* dims, int32_t rank, const char* dformat);

/* One pass over the kernels with inputs already resident on the device. */
int32_t ogle_rt_compute(OgleSession* s);
/* The same pass as one captured hipGraph (captured on the first call). */
int32_t ogle_rt_compute_graph(OgleSession* s);
int32_t ogle_rt_sync(OgleSession* s);
/* 1 if graph slot `slot` (0 or 1) holds a recorded pass, 0 if not.  Loading a graph
 * into a session drops every recorded pass of the previous one. */
int32_t ogle_rt_graph_captured(OgleSession* s, int32_t slot);

/*
 * The executor's dependency rule on plain data (touches no device): 1 if a launch that
 * reads the byte ranges [read_ptrs[i], +read_bytes[i]) and writes [write_ptrs[i],
 * +write_bytes[i]) must wait for one of the `n_pending` deferred convolutions, i.e. a
 * read overlaps something one of them writes (output, workspace) or a write overlaps
 * anything one of them reads or writes; 0 otherwise.  The reference needs no such rule
 * (one draw per node, in order, fbo_session.cc:140-153); here convolutions are held
 * back to share grids, and this is what decides when they must go out.
 */
int32_t ogle_rt_hazard_conflicts(const OgleConvArgs* pending, int32_t n_pending,
                                 const void* const* read_ptrs, const size_t* read_bytes,
                                 int32_t n_reads, const void* const* write_ptrs,
                                 const size_t* write_bytes, int32_t n_writes);

/* The same rule for a convolution as the next launch: what `next` reads (input, filter,
 * bias) and writes (output(s), workspace; with out_image_stride one range per image, so
 * that convolutions whose images interleave inside one tensor do not count as
 * overlapping) against the `n_pending` deferred ones. */
int32_t ogle_rt_conv_hazard_conflicts(const OgleConvArgs* pending, int32_t n_pending,
                                      const OgleConvArgs* next);

/*
 * Times `iters` passes (after `warmup` untimed ones) with HIP events recorded on
 * the session's stream; inputs stay resident.  use_graph selects ogle_rt_compute
 * or ogle_rt_compute_graph; with_detect appends the SSD decode + score-filter launch
 * (Detector's device stage, default tensor names and thresholds) to every pass;
 * sync_each waits for each pass before enqueuing the next (latency mode).
 * ms_each (may be NULL) receives one duration per pass, each pass bracketed by its
 * own event pair; *total_ms the span of all passes.
 */
int32_t ogle_rt_time_compute(OgleSession* s, int32_t warmup, int32_t iters, int32_t use_graph,
                             int32_t with_detect, int32_t sync_each, float* ms_each,
                             float* total_ms);

/*
 * Throughput of `n` sessions that hold the same graph, run as a pipeline: every session
 * replays its pass (network, and with_detect the detector's device work) as a hipGraph
 * on its own stream, and `iters` passes are dealt round-robin over the sessions from the
 * calling thread, so that one session's launch gaps and under-filled kernels are
 * covered by the others' work.  Each session must have run once (inputs resident).
 * `warmup` untimed passes first; total_ms is the time from the common start (all
 * streams idle) until the last stream is idle again.  The reference executes one
 * graph on one GL context (fbo_session.cc:127-153); this is what a server that keeps
 * several batches in flight does with it.
 *
 * host_inputs == NULL: the inputs stay resident.  Otherwise host_inputs[i] is a host
 * buffer with the bytes of session i's input tensor `input_name` (dense NHWC fp32, as
 * FBOSession::Run takes it) and every pass starts with its asynchronous copy to the
 * device on that session's stream, so uploads overlap the other sessions' kernels.
 * The copies are only asynchronous from page-locked memory (ogle_rt_alloc_pinned).
 */
int32_t ogle_rt_time_pipelined(OgleSession** sessions, int32_t n, int32_t warmup, int32_t iters,
                               int32_t with_detect, const char* input_name,
                               const void* const* host_inputs, float* total_ms);

/* Page-locked host memory (hipHostMalloc / hipHostFree); NULL when it cannot be had. */
void* ogle_rt_alloc_pinned(size_t bytes);
void ogle_rt_free_pinned(void* p);

/*
 * One pass with an event pair around every node (the reference's per-node TraceMe
 * with sync, fbo_session.cc:140-153).  Returns the number of nodes timed, or a
 * negative status.  ogle_rt_profile_entry then reads entry i: its
 * "<node>#<type>#" label, op type and milliseconds.
 */
int32_t ogle_rt_profile(OgleSession* s);
int32_t ogle_rt_profile_entry(OgleSession* s, int32_t i, const char** label, const char** type,
                              float* ms);

/*
 * Dispatch sequence of a pass.  ogle_rt_launch_plan makes one eager pass (with_detect:
 * followed by the detector's device work) and records, in issue order, every call into the
 * kernel library with the node(s) it was made for and the number of device operations it
 * became; it returns the number of entries.  ogle_rt_launch_plan_entry reads entry i: its
 * label ("<node>#<type>#", the reference's TraceMe label, fbo_session.cc:140-153; the
 * nodes of convolutions that went out as one batch are joined with '+'; "reduce:" marks
 * the grid that finishes their split-K reductions), its dispatch count, and the duration
 * of each of its device operations in that pass (up to `capacity` values), taken from
 * events the device stamps with the kernel's own begin and end
 * (ogle_hip_kernel_timing_begin).  A replayed hipGraph of the pass issues exactly this
 * sequence, so a profiler's kernel trace of the replays can be attributed to layers
 * position by position, and the durations here are the same quantity that trace shows.
 */
int32_t ogle_rt_launch_plan(OgleSession* s, int32_t with_detect);
int32_t ogle_rt_launch_plan_entry(OgleSession* s, int32_t i, const char** label,
                                  int32_t* dispatches, float* microseconds, int32_t capacity);

/* Shape of a tensor by name (FindTensorByName): writes up to 8 dims, returns rank. */
int32_t ogle_rt_tensor_shape(OgleSession* s, const char* name, int32_t* dims);
/* Layout tag of a tensor as a TensorProto.DataFormat value (dlxnet.proto:7-30), or negative. */
int32_t ogle_rt_tensor_dformat(OgleSession* s, const char* name);
/* Device address of a tensor's first element (for zero-copy consumers), or NULL; NULL too
 * for a tensor that is not dense on the device (a convolution output produced in its place
 * inside a concatenation's output at batch > 1: read it with ogle_rt_get_output). */
void* ogle_rt_tensor_device_ptr(OgleSession* s, const char* name);
/* The session's hipStream_t. */
void* ogle_rt_stream(OgleSession* s);

/*
 * FBOSession::GetOutputs for one tensor (fbo_session.cc:276-300): copies it to
 * `dst` (capacity in floats) converted to `dformat`; the sync point.  Returns the
 * element count.
 */
int64_t ogle_rt_get_output(OgleSession* s, const char* name, const char* dformat, float* dst,
                           int64_t capacity);

/*
 * Parses a serialized ModelProto with the runtime's own wire codec and serializes
 * it again into `out` (capacity bytes): returns the size written, or negative.  Lets
 * a test check the hand-written .dlx codec against another protobuf implementation.
 * ogle_rt_model_debug_string does the same into the text form of DebugString().
 */
int64_t ogle_rt_reserialize(const void* data, size_t size, void* out, int64_t capacity);
int64_t ogle_rt_model_debug_string(const void* data, size_t size, char* out, int64_t capacity);

/* Number of kernels the loaded graph created, and registered op-type names. */
int32_t ogle_rt_num_kernels(OgleSession* s);

/*
 * Issue order.  The reference runs nodes in file order (fbo_session.cc:140-153), and so
 * does a session here unless ogle_rt_set_reorder(s, 1) is called before the first run:
 * then a convolution whose result is not needed at once may be issued earlier, next
 * to another one, so that both share a grid (same results).  ogle_rt_issue_order_name returns the name of
 * the i-th node a pass issues (valid after the first run; NULL past the end).
 */
int32_t ogle_rt_set_reorder(OgleSession* s, int32_t on);
/*
 * Sibling fusion.  Two Conv nodes that read the same tensor with the same attributes (the
 * box and the class head of an SSD feature map) run as one launch that fetches the input
 * once and writes each node's channels to its own tensor; the reference draws them one
 * after the other.  Off by default (one launch per node); ogle_rt_set_fuse_siblings(s, 1)
 * before the first run switches it on.  Results agree to summation order.
 */
int32_t ogle_rt_set_fuse_siblings(OgleSession* s, int32_t on);
const char* ogle_rt_issue_order_name(OgleSession* s, int32_t i);
int32_t ogle_rt_registered_kernel_count(void);
const char* ogle_rt_registered_kernel_name(int32_t i);

/* One detection, as BoxInfo (examples/ssd/common.h:29-45). */
typedef struct OgleDetection {
  int32_t image;      /* index in the batch */
  int32_t prior;      /* BoxInfo.index */
  int32_t class_id;   /* BoxInfo.class_name */
  float score;
  int32_t x, y, width, height; /* BoxInfo.box (integer rectangle) */
  float cx, cy;
} OgleDetection;

/*
 * Detector::Detect (examples/ssd/detector.cc:275-295) on a loaded session: runs the
 * graph on `images` (host NHWC floats, already preprocessed), decodes and filters
 * on the device, then top-k and NMS (device or host, ogle_rt_set_device_nms).  Tensor names are cls_logits / box_preds /
 * anchors unless overridden (NULL keeps the default).  Writes up to `capacity`
 * detections, returns how many there are in total.
 */
/* Top-k + NMS of ogle_rt_detect / ogle_rt_time_compute on the device (default, 1) or on
 * the host as in the reference (0).  Same detections either way. */
int32_t ogle_rt_set_device_nms(OgleSession* s, int32_t on);

int64_t ogle_rt_detect(OgleSession* s, const float* images, const int32_t* dims /* n,h,w,c */,
                       const char* input_name, const char* cls_name, const char* box_name,
                       const char* anchors_name, float score_threshold, float nms_threshold,
                       int32_t topk, int32_t raw_width, int32_t raw_height, OgleDetection* out,
                       int64_t capacity);

/*
 * The detections of the detector work most recently enqueued on the session's
 * stream (by ogle_rt_time_compute with with_detect, eagerly or inside its graph):
 * waits for the stream, reads the lists back and, with host NMS selected, finishes
 * them on the host.  Same output convention as ogle_rt_detect.
 */
int64_t ogle_rt_detect_results(OgleSession* s, OgleDetection* out, int64_t capacity);

/*
 * ogle_rt_time_pipelined with the detector's work in every pass, and the host in the loop:
 * every pass ends with ONE asynchronous copy of its final detection lists (a count and at
 * most top-k records of 44 bytes per image, one device block) into page-locked host
 * memory, recorded inside the captured graph.  The host never waits for a stream: before a
 * session's next pass is launched it waits for the event behind that session's previous
 * pass and reads its lists, while the other sessions' passes (and, with one session, nothing)
 * are already enqueued.  `detections` receives the number of detections read in the timed
 * passes.  The reference's timing loop reads its outputs back inside every run as well
 * (nn/main.cc:76-111).  Needs top-k + NMS on the device (the default).
 */
int32_t ogle_rt_time_pipelined_readback(OgleSession** sessions, int32_t n, int32_t warmup,
                                        int32_t iters, float* total_ms, int64_t* detections);
/* The detections of the session's last pass launched by ogle_rt_time_pipelined_readback,
 * read from the page-locked copy (waits for that pass's event if nobody has yet).  Same
 * output convention as ogle_rt_detect. */
int64_t ogle_rt_pipelined_results(OgleSession* s, OgleDetection* out, int64_t capacity);

#ifdef __cplusplus
}
#endif

#endif /* OGLE_RUNTIME_H_ */
