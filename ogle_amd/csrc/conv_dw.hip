// Depthwise convolution over NHWC (group == C_in == C_out, multiplier 1).
// Bandwidth bound (about 2 FLOP per byte): the kernel is organised around
// reading every input element from HBM once and writing every output once.
//
// Thread mapping: consecutive threads take consecutive 16-byte channel vectors
// of consecutive pixel columns of one image row, so a wave's loads and stores
// are contiguous runs of NHWC memory.  Each thread owns a small patch of output
// pixels (R rows x Q columns) and requests every input vector the patch needs
// with branch-free buffer loads before it starts to accumulate, so all of a
// wave's loads are in flight at once; neighbouring patches' halo vectors are the
// same bytes other lanes and the adjacent wave load at the same time and are
// served by the vector L1 / the XCD's L2 (the block order keeps neighbours on one
// XCD).
//
// Semantics follow conv2d_dw.glsl:38-96: accumulator starts at the bias, taps
// outside the image are skipped, order ky then kx, then the fused activation.
// Filter layout: [k*k][C] (tap major) so a thread's taps are contiguous vectors.
#include "common.h"

namespace ogle {
namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct Vec;
template <>
struct Vec<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ static void unpack(const u32x4& t, float (&v)[4]) {
    v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y);
    v[2] = __uint_as_float(t.z); v[3] = __uint_as_float(t.w);
  }
  __device__ static void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
  __device__ static u32x4 pack(const float (&v)[4]) {
    u32x4 t;
    t.x = __float_as_uint(v[0]); t.y = __float_as_uint(v[1]);
    t.z = __float_as_uint(v[2]); t.w = __float_as_uint(v[3]);
    return t;
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
  __device__ static void unpack(const u32x4& t, float (&v)[8]) {
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
  __device__ static u32x4 pack(const float (&v)[8]) {
    u32x4 t;
    __half2* h = reinterpret_cast<__half2*>(&t);
#pragma unroll
    for (int i = 0; i < 4; ++i) h[i] = __floats2half2_rn(v[2 * i], v[2 * i + 1]);
    return t;
  }
};

// Unsigned division by a number fixed at launch: q = (mulhi(n, mul) + n) >> shift,
// exact for every n below 2^31 (Granlund and Montgomery's round-up form).
struct FastDiv {
  unsigned mul, shift, d;
};

__device__ __forceinline__ unsigned fast_div(unsigned n, const FastDiv& f) {
  return (__umulhi(n, f.mul) + n) >> f.shift;
}

// 3x3, dilation 1, stride S, channel count a multiple of the vector width.
// A thread owns a patch of R output rows x Q output columns of one channel vector.
// Index arithmetic is kept off the vector ALU as far as possible (the kernel issues
// about as many address instructions as FMAs otherwise): the thread index is split
// with multiply-high divisions, input offsets are a row term plus a column term, and
// a tap outside the image just gets the out-of-range bit set in its offset.
template <typename T, int S, int R, int Q>
__global__ __launch_bounds__(256) void dwconv3x3_strip(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ y, int h, int wd, int c, int oh, int ow, int pad, Epilogue ep,
    unsigned x_bytes, unsigned y_bytes, unsigned total, FastDiv div_cv, FastDiv div_cols,
    FastDiv div_strips) {
  constexpr int V = Vec<T>::N;
  constexpr int IN_ROWS = (R - 1) * S + 3;
  constexpr int IN_COLS = (Q - 1) * S + 3;
  constexpr unsigned ESZ = sizeof(T);
  constexpr unsigned kOut = 0x80000000u;  // offsets at or above this are outside every operand
  // Consecutive logical blocks (neighbouring pixels and strips, which share halo
  // rows) are kept on one XCD so that the re-read rows hit that XCD's L2.
  const unsigned idx = (unsigned)xcd_swizzle(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (idx >= total) return;
  const unsigned t1 = fast_div(idx, div_cv);
  const int cg = (int)(idx - t1 * div_cv.d);
  const unsigned t2 = fast_div(t1, div_cols);
  const int oxg = (int)(t1 - t2 * div_cols.d);
  const unsigned b = fast_div(t2, div_strips);
  const int strip = (int)(t2 - b * div_strips.d);
  const int ch = cg * V;
  const int oy0 = strip * R;
  const int ox0 = oxg * Q;

  float wt[9][V];
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) Vec<T>::load(w + tap * c + ch, wt[tap]);

  float acc[R][Q][V];
  {
    float bv[V];
#pragma unroll
    for (int v = 0; v < V; ++v) bv[v] = 0.f;
    if (bias != nullptr) {
#pragma unroll
      for (int v = 0; v < V; v += 4) {
        const float4 t = *reinterpret_cast<const float4*>(bias + ch + v);  // ch % 4 == 0
        bv[v] = t.x; bv[v + 1] = t.y; bv[v + 2] = t.z; bv[v + 3] = t.w;
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int q = 0; q < Q; ++q)
#pragma unroll
        for (int v = 0; v < V; ++v) acc[r][q][v] = bv[v];
  }

  // Every input vector the patch needs is requested up front with buffer loads;
  // taps outside the image get an out-of-range offset and come back as zeros, so
  // there is no branch between the loads and they are all in flight together.
  const int iy0 = oy0 * S - pad;
  const int ix0 = ox0 * S - pad;
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(x), 0, (int)x_bytes, 0x00020000);
  const unsigned row_bytes = (unsigned)(wd * c) * ESZ;
  const unsigned img = (b * (unsigned)h) * row_bytes + (unsigned)ch * ESZ;
  unsigned row_off[IN_ROWS], col_off[IN_COLS];
#pragma unroll
  for (int j = 0; j < IN_ROWS; ++j) {
    const int iy = iy0 + j;
    row_off[j] = (unsigned)iy < (unsigned)h ? img + (unsigned)iy * row_bytes : kOut;
  }
#pragma unroll
  for (int s = 0; s < IN_COLS; ++s) {
    const int ix = ix0 + s;
    col_off[s] = (unsigned)ix < (unsigned)wd ? (unsigned)(ix * c) * ESZ : kOut;
  }
  u32x4 raw[IN_ROWS][IN_COLS];
#pragma unroll
  for (int j = 0; j < IN_ROWS; ++j)
#pragma unroll
    for (int s = 0; s < IN_COLS; ++s) {
      // a valid row plus a valid column stays below 2^31; either term being kOut sets
      // the top bit of the OR, whatever the sum wrapped to
      const unsigned off = (row_off[j] + col_off[s]) | ((row_off[j] | col_off[s]) & kOut);
      raw[j][s] = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)off, 0, 0);
    }
#pragma unroll
  for (int j = 0; j < IN_ROWS; ++j) {
    float in[IN_COLS][V];
#pragma unroll
    for (int s = 0; s < IN_COLS; ++s) Vec<T>::unpack(raw[j][s], in[s]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int ky = j - r * S;  // compile-time after unrolling
      if (ky < 0 || ky > 2) continue;
#pragma unroll
      for (int q = 0; q < Q; ++q) {
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
#pragma unroll
          for (int v = 0; v < V; ++v) acc[r][q][v] += wt[ky * 3 + kx][v] * in[q * S + kx][v];
        }
      }
    }
  }
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(y, 0, (int)y_bytes, 0x00020000);
  const unsigned out_row_bytes = (unsigned)(ow * c) * ESZ;
  const unsigned out0 = (b * (unsigned)oh + (unsigned)oy0) * out_row_bytes +
                        (unsigned)(ox0 * c + ch) * ESZ;
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      float out[V];
#pragma unroll
      for (int v = 0; v < V; ++v) out[v] = apply_epilogue(acc[r][q][v], ep);
      const bool ok = oy0 + r < oh && ox0 + q < ow;
      const unsigned off = ok ? out0 + (unsigned)r * out_row_bytes + (unsigned)(q * c) * ESZ : kOut;
      __builtin_amdgcn_raw_buffer_store_b128(Vec<T>::pack(out), ry, (int)off, 0, 0);
    }
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

FastDiv make_fast_div(unsigned d) {
  FastDiv f{0, 0, d};
  unsigned l = 0;
  while ((1ull << l) < d) ++l;
  f.shift = l;
  f.mul = (unsigned)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
  return f;
}

template <typename T, int S, int R, int Q = 1>
int32_t launch_strip(const OgleConvArgs& a, hipStream_t s, const Epilogue& ep) {
  constexpr int V = Vec<T>::N;
  const int strips = (a.out_h + R - 1) / R, cols = (a.out_w + Q - 1) / Q, cv = a.in_c / V;
  const long total = (long)a.n * strips * cols * cv;
  const int blocks = (ceil_div(total, 256) + 7) / 8 * 8;  // whole XCD rounds
  hipLaunchKernelGGL((dwconv3x3_strip<T, S, R, Q>), dim3(blocks), dim3(256), 0, s,
                     static_cast<const T*>(a.input_dev), static_cast<const T*>(a.filter_dev),
                     a.bias_dev, static_cast<T*>(a.output_dev), a.in_h, a.in_w, a.in_c, a.out_h,
                     a.out_w, a.padding, ep,
                     (unsigned)((long)a.n * a.in_h * a.in_w * a.in_c * sizeof(T)),
                     (unsigned)((long)a.n * a.out_h * a.out_w * a.in_c * sizeof(T)), (unsigned)total,
                     make_fast_div((unsigned)cv), make_fast_div((unsigned)cols),
                     make_fast_div((unsigned)strips));
  return check_launch("dwconv3x3_strip");
}

template <typename T, int S>
int32_t pick_strip(const OgleConvArgs& a, hipStream_t s, const Epilogue& ep) {
  constexpr int V = Vec<T>::N;
  // A 2x2 (stride 1) or 2x1 patch per thread shares input rows and columns in
  // registers; smaller problems fall back to one output per thread so that the
  // grid still covers the 256 CUs (measured on MI355X: patches beyond 2 rows gain
  // nothing once all loads of a patch are in flight together).
  const long per_row_threads = (long)a.n * a.out_w * (a.in_c / V);
  const long want = 256L * 256 * 4;
  if (S == 1 && per_row_threads / 2 * ((a.out_h + 1) / 2) >= want / 2)
    return launch_strip<T, S, 2, 2>(a, s, ep);
  if (per_row_threads * ((a.out_h + 1) / 2) >= want / 2) return launch_strip<T, S, 2, 1>(a, s, ep);
  return launch_strip<T, S, 1>(a, s, ep);
}

template <typename T>
int32_t run_dw(const OgleConvArgs& a, hipStream_t s) {
  const Epilogue ep = make_epilogue(a.act, a.min_value, a.max_value, a.act_variant);
  constexpr int V = Vec<T>::N;
  // the strip kernel addresses the input with 32-bit byte offsets (buffer loads)
  // and the bias with 16-byte loads
  const bool fits = (long)a.n * a.in_h * a.in_w * a.in_c * (long)sizeof(T) < 0x7fffffffL &&
                    (long)a.n * a.out_h * a.out_w * a.in_c * (long)sizeof(T) < 0x7fffffffL &&
                    (reinterpret_cast<uintptr_t>(a.bias_dev) & 15u) == 0;
  if (a.kernel_size == 3 && a.dilation == 1 && a.in_c % V == 0 && fits &&
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
