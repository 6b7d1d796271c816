// Shared device/host helpers for the gfx950 kernels.
#ifndef OGLE_CSRC_COMMON_H_
#define OGLE_CSRC_COMMON_H_

#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ogle_hip.h"

namespace ogle {

// Thread-local message for ogle_hip_last_error().
void set_error(const char* fmt, ...);

inline int32_t fail(int32_t status, const char* what) {
  set_error("%s", what);
  return status;
}

// Reports the launch status of the kernel just enqueued (and counts it for
// ogle_hip_launch_count).
int32_t check_launch(const char* kernel);
// Counts a device operation that is not one of the library's kernels (a copy).
void note_launch();

inline hipStream_t as_stream(ogle_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Kernel timing (ogle_hip_kernel_timing_begin / _end): while it is on for the calling
// thread, every kernel is launched with a start and a stop event of its own, which the
// runtime stamps with the kernel's own begin and end on the device.  next_timing_events
// hands out the pair for the next launch, or returns false when timing is off.
bool next_timing_events(hipEvent_t* start, hipEvent_t* stop);

// Every kernel of the library is launched through this.
template <typename F, typename... Args>
inline void launch(F kernel, const dim3& grid, const dim3& block, unsigned shared_bytes,
                   hipStream_t stream, Args... args) {
  hipEvent_t e0, e1;
  if (next_timing_events(&e0, &e1)) {
    hipExtLaunchKernelGGL(kernel, grid, block, shared_bytes, stream, e0, e1, 0, args...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, shared_bytes, stream, args...);
  }
}

inline int ceil_div(long a, long b) { return static_cast<int>((a + b - 1) / b); }

// Fused activation with the variant rules of the reference's shaders
// (conv2d.glsl:82-90, conv2d_pw.glsl:82-90, conv2d_any4.glsl:89-94).  The
// bounds are resolved on the host into (lo, hi) plus two flags so that the
// device code is variant free.
struct Epilogue {
  float lo;
  float hi;
  int use_lo;
  int use_hi;
};

inline Epilogue make_epilogue(int act, float minv, float maxv, int variant) {
  Epilogue e{0.f, 0.f, 0, 0};
  if (act == OGLE_ACT_CLIP) {
    e.lo = (variant == OGLE_VARIANT_PW) ? 0.f : minv;
    e.hi = maxv;
    e.use_lo = 1;
    e.use_hi = 1;
  } else if (act == OGLE_ACT_RELU) {
    e.lo = (variant == OGLE_VARIANT_ANY4) ? minv : 0.f;
    e.use_lo = 1;
  }
  return e;
}

__device__ __forceinline__ float apply_epilogue(float v, const Epilogue& e) {
  if (e.use_lo) v = v < e.lo ? e.lo : v;
  if (e.use_hi) v = v > e.hi ? e.hi : v;
  return v;
}

// Storage <-> fp32 conversions.
__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(__half v) { return __half2float(v); }
template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ __half from_f32<__half>(float v) { return __float2half_rn(v); }


// Result stores.  A kernel's results are written through to memory (system scope) while it
// runs.  Left dirty in the L2s they are all written back at the end of the kernel, when
// nothing is left to overlap the write-back with; measured on MI355X the depthwise layers
// of the network are 7 % faster this way, the fp16 GEMM of 12 GFLOP 13 %, a whole batch-16
// pass 1.5 %.  (Non-temporal stores were slower than plain ones.)
constexpr int kResultStoreAux = 17;   // raw buffer stores: sc0 | sc1
__device__ __forceinline__ void store_result16(void* dst, float4 v) {
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  const f32x4_t t = {v.x, v.y, v.z, v.w};
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(dst), "v"(t) : "memory");
}
__device__ __forceinline__ void store_result16(void* dst, uint4 v) {
  typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t t = {v.x, v.y, v.z, v.w};
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(dst), "v"(t) : "memory");
}
__device__ __forceinline__ void store_result8(void* dst, uint2 v) {
  typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
  const u32x2_t t = {v.x, v.y};
  asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" ::"v"(dst), "v"(t) : "memory");
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.
// Remaps the linear workgroup id so that consecutive logical ids land on the
// same XCD, keeping tiles that share operands in one L2.
__device__ __forceinline__ int xcd_swizzle(int pid, int grid) {
  constexpr int kXcds = 8;
  if (grid % kXcds != 0) return pid;
  return (pid % kXcds) * (grid / kXcds) + pid / kXcds;
}

// Launchers implemented in the .hip files (host side).
int32_t launch_conv_igemm(const OgleConvArgs& a, hipStream_t s);   // returns OGLE_ERR_UNSUPPORTED if shape not eligible
size_t conv_igemm_workspace_bytes(const OgleConvArgs& a);
bool conv_igemm_takes(const OgleConvArgs& a);  // launch_conv_igemm would not return OGLE_ERR_UNSUPPORTED
int32_t launch_conv_igemm_static_scratch(const OgleConvArgs& a, hipStream_t s);
// fp16-storage pointwise GEMM with operands streamed straight into LDS: the tile
// configuration it would run `a` with, or -1 if it does not take the shape.
int f16_async_config(const OgleConvArgs& a);
int32_t launch_pw_gemm_f16_async(const OgleConvArgs& a, hipStream_t s);
// reduce_pending != nullptr: split-K reductions are not launched; reduce_pending[i] says
// whether convolution i still needs launch_conv_reduce.
int32_t launch_conv_batch(const OgleConvArgs* args, int count, hipStream_t s,
                          int32_t (*fallback)(const OgleConvArgs&, hipStream_t),
                          int32_t* reduce_pending = nullptr);
int32_t launch_conv_reduce(const OgleConvArgs* args, int count, hipStream_t s);
int32_t launch_conv_direct(const OgleConvArgs& a, hipStream_t s);
int32_t launch_conv_dw(const OgleConvArgs& a, hipStream_t s);
int32_t launch_pool(const OglePoolArgs& a, hipStream_t s);
int32_t launch_concat(const OgleConcatArgs& a, hipStream_t s);
int32_t launch_transpose(const OgleTransposeArgs& a, hipStream_t s);
int32_t launch_decode(const OgleDecodeArgs& a, hipStream_t s);
int32_t launch_detect(const OgleDetectArgs& a, hipStream_t s);
int32_t launch_unary(const OgleUnaryArgs& a, hipStream_t s);
int32_t launch_binary(const OgleBinaryArgs& a, hipStream_t s);
int32_t launch_batchnorm(const OgleBatchNormArgs& a, hipStream_t s);
int32_t launch_gemm(const OgleGemmArgs& a, hipStream_t s);
size_t gemm_workspace_bytes(const OgleGemmArgs& a);
int32_t launch_topk_nms(const OgleNmsArgs& a, hipStream_t s);
size_t topk_nms_lds_bytes(int stride, int topk);
int32_t launch_expf(const float* x, float* y, int64_t n, hipStream_t s);
int32_t launch_pack_filter(const float* src, void* dst, int layout, int dtype, int o, int i,
                           int kh, int kw, hipStream_t s);
int32_t launch_convert(const void* src, int sdt, void* dst, int ddt, int64_t n, hipStream_t s);

}  // namespace ogle

#endif  // OGLE_CSRC_COMMON_H_
