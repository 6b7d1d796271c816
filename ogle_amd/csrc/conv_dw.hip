// Depthwise convolution over NHWC (group == C_in == C_out, multiplier 1).
// Bandwidth bound (about 2 FLOP per byte): the kernel is organised around
// reading every input element from HBM once and writing every output once.
//
// Thread mapping: consecutive threads take consecutive 16-byte channel vectors
// of consecutive pixels of one image row, so a wave's loads and stores are
// contiguous runs of NHWC memory.  Each thread owns a vertical strip of R
// output rows and walks the input rows the strip needs once, so vertically
// adjacent outputs share their input rows in registers; the horizontal
// neighbours (x-1, x+1) are the same bytes other lanes of the same and the
// adjacent wave load at the same time and are served by the vector L1.
//
// Semantics follow conv2d_dw.glsl:38-96: accumulator starts at the bias, taps
// outside the image are skipped, order ky then kx, then the fused activation.
// Filter layout: [k*k][C] (tap major) so a thread's taps are contiguous vectors.
#include "common.h"

namespace ogle {
namespace {

template <typename T>
struct Vec;
template <>
struct Vec<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ static void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <>
struct Vec<__half> {
  static constexpr int N = 8;
  __device__ static void load(const __half* p, float (&v)[8]) {
    const uint4 t = *reinterpret_cast<const uint4*>(p);
    const __half2* h = reinterpret_cast<const __half2*>(&t);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float2 f = __half22float2(h[i]);
      v[2 * i] = f.x;
      v[2 * i + 1] = f.y;
    }
  }
  __device__ static void store(__half* p, const float (&v)[8]) {
    uint4 t;
    __half2* h = reinterpret_cast<__half2*>(&t);
#pragma unroll
    for (int i = 0; i < 4; ++i) h[i] = __floats2half2_rn(v[2 * i], v[2 * i + 1]);
    *reinterpret_cast<uint4*>(p) = t;
  }
};

// 3x3, dilation 1, stride S, channel count a multiple of the vector width.
template <typename T, int S, int R>
__global__ __launch_bounds__(256) void dwconv3x3_strip(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ y, int n, int h, int wd, int c, int oh, int ow, int pad, Epilogue ep) {
  constexpr int V = Vec<T>::N;
  constexpr int IN_ROWS = (R - 1) * S + 3;
  const int cv = c / V;
  const int strips = (oh + R - 1) / R;
  const long total = (long)n * strips * ow * cv;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int cg = (int)(idx % cv);
  long t = idx / cv;
  const int ox = (int)(t % ow);
  t /= ow;
  const int strip = (int)(t % strips);
  const int b = (int)(t / strips);
  const int ch = cg * V;
  const int oy0 = strip * R;

  float wt[9][V];
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) Vec<T>::load(w + (long)tap * c + ch, wt[tap]);

  float acc[R][V];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int v = 0; v < V; ++v) acc[r][v] = bias != nullptr ? bias[ch + v] : 0.f;

  const int iy0 = oy0 * S - pad;
  const int ix0 = ox * S - pad;
  const T* xb = x + (long)b * h * wd * c + ch;
#pragma unroll
  for (int j = 0; j < IN_ROWS; ++j) {
    const int iy = iy0 + j;
    if (iy < 0 || iy >= h) continue;
    float in[3][V];
    bool ok[3];
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      const int ix = ix0 + s;
      ok[s] = ix >= 0 && ix < wd;
      if (ok[s]) Vec<T>::load(xb + ((long)iy * wd + ix) * c, in[s]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int ky = j - r * S;  // compile-time after unrolling
      if (ky < 0 || ky > 2) continue;
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        if (!ok[s]) continue;
#pragma unroll
        for (int v = 0; v < V; ++v) acc[r][v] += wt[ky * 3 + s][v] * in[s][v];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int oy = oy0 + r;
    if (oy >= oh) break;
    float out[V];
#pragma unroll
    for (int v = 0; v < V; ++v) out[v] = apply_epilogue(acc[r][v], ep);
    Vec<T>::store(y + (((long)b * oh + oy) * ow + ox) * c + ch, out);
  }
}

// Any kernel size / dilation / channel count: one thread per output element.
template <typename T>
__global__ __launch_bounds__(256) void dwconv_general(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ y, int n, int h, int wd, int c, int oh, int ow, int k, int stride, int pad,
    int dil, Epilogue ep) {
  const long total = (long)n * oh * ow * c;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int ch = (int)(idx % c);
    long pix = idx / c;
    const int ox = (int)(pix % ow);
    pix /= ow;
    const int oy = (int)(pix % oh);
    const int b = (int)(pix / oh);
    float acc = bias != nullptr ? bias[ch] : 0.f;
    for (int r = 0; r < k; ++r) {
      const int iy = oy * stride - pad + r * dil;
      if (iy < 0 || iy >= h) continue;
      for (int s = 0; s < k; ++s) {
        const int ix = ox * stride - pad + s * dil;
        if (ix < 0 || ix >= wd) continue;
        acc += to_f32(w[(long)(r * k + s) * c + ch]) *
               to_f32(x[(((long)b * h + iy) * wd + ix) * c + ch]);
      }
    }
    y[idx] = from_f32<T>(apply_epilogue(acc, ep));
  }
}

template <typename T, int S, int R>
int32_t launch_strip(const OgleConvArgs& a, hipStream_t s, const Epilogue& ep) {
  constexpr int V = Vec<T>::N;
  const long total = (long)a.n * ((a.out_h + R - 1) / R) * a.out_w * (a.in_c / V);
  const int blocks = ceil_div(total, 256);
  hipLaunchKernelGGL((dwconv3x3_strip<T, S, R>), dim3(blocks), dim3(256), 0, s,
                     static_cast<const T*>(a.input_dev), static_cast<const T*>(a.filter_dev),
                     a.bias_dev, static_cast<T*>(a.output_dev), a.n, a.in_h, a.in_w, a.in_c,
                     a.out_h, a.out_w, a.padding, ep);
  return check_launch("dwconv3x3_strip");
}

template <typename T, int S>
int32_t pick_strip(const OgleConvArgs& a, hipStream_t s, const Epilogue& ep) {
  constexpr int V = Vec<T>::N;
  // Taller strips reuse more input rows in registers but cut the thread count;
  // keep at least ~4 waves per SIMD's worth of threads on the 256 CUs.
  const long per_row_threads = (long)a.n * a.out_w * (a.in_c / V);
  const long want = 256L * 256 * 4;
  if (per_row_threads * ((a.out_h + 3) / 4) >= want) return launch_strip<T, S, 4>(a, s, ep);
  if (per_row_threads * ((a.out_h + 1) / 2) >= want) return launch_strip<T, S, 2>(a, s, ep);
  return launch_strip<T, S, 1>(a, s, ep);
}

template <typename T>
int32_t run_dw(const OgleConvArgs& a, hipStream_t s) {
  const Epilogue ep = make_epilogue(a.act, a.min_value, a.max_value, a.act_variant);
  constexpr int V = Vec<T>::N;
  if (a.kernel_size == 3 && a.dilation == 1 && a.in_c % V == 0 &&
      (a.stride == 1 || a.stride == 2)) {
    if (a.stride == 1) return pick_strip<T, 1>(a, s, ep);
    return pick_strip<T, 2>(a, s, ep);
  }
  const long total = (long)a.n * a.out_h * a.out_w * a.out_c;
  int blocks = ceil_div(total, 256);
  if (blocks > 256 * 64) blocks = 256 * 64;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((dwconv_general<T>), dim3(blocks), dim3(256), 0, s,
                     static_cast<const T*>(a.input_dev), static_cast<const T*>(a.filter_dev),
                     a.bias_dev, static_cast<T*>(a.output_dev), a.n, a.in_h, a.in_w, a.in_c,
                     a.out_h, a.out_w, a.kernel_size, a.stride, a.padding, a.dilation, ep);
  return check_launch("dwconv_general");
}

}  // namespace

int32_t launch_conv_dw(const OgleConvArgs& a, hipStream_t s) {
  if (a.dtype == OGLE_F16) return run_dw<__half>(a, s);
  return run_dw<float>(a, s);
}

}  // namespace ogle
