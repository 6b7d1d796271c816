// Depthwise convolution over NHWC (group == C_in == C_out, multiplier 1).
// Bandwidth bound (about 2 FLOP per byte): the kernel is organised around
// reading every input element from HBM once and writing every output once.
//
// Thread mapping: consecutive threads take consecutive 16-byte channel vectors
// of consecutive pixel columns of one image row, so a wave's loads and stores
// are contiguous runs of NHWC memory.  A thread walks down a segment of output rows
// with the input rows it needs in a ring of registers and the next rows already
// requested (see dwconv3x3_rows); neighbouring threads' halo columns are the same
// bytes other lanes and the adjacent wave load at the same time and are served by
// the vector L1 / the XCD's L2 (the block order keeps neighbours on one XCD).
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

// 3x3, dilation 1, stride S, channel count a multiple of the vector width.  A thread owns Q output columns of one
// channel vector and walks DOWN a segment of output rows, holding the input rows it needs
// in a ring of registers: moving one output row down re-uses 3 - S of the 3 input rows and
// loads S new ones, so an input vector is requested once per thread that needs it (2
// requests per output at stride 1 with Q = 2, against 4 for a 2x2 patch and 9 naively),
// and the rows PF steps ahead are requested before the current row is accumulated: the
// loads of a wave never stop while it computes and stores.  Rows above / below the image
// and columns left / right of it come back as zeros (out-of-range buffer offsets), rows
// past the end of the segment are not requested at all.
template <typename T, int S, int Q, int PF>
__global__ __launch_bounds__(256) void dwconv3x3_rows(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ y, int h, int wd, int c, int oh, int ow, int pad, Epilogue ep,
    unsigned x_bytes, unsigned y_bytes, unsigned total, FastDiv div_cv, FastDiv div_cols,
    FastDiv div_segs, int seg_rows) {
  constexpr int V = Vec<T>::N;
  constexpr int IN_COLS = (Q - 1) * S + 3;
  constexpr int NB = 3 + S * PF;  // ring of input rows: three in use, S * PF on their way
  constexpr unsigned ESZ = sizeof(T);
  constexpr unsigned kOut = 0x80000000u;
  const unsigned idx = (unsigned)xcd_swizzle(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (idx >= total) return;
  const unsigned t1 = fast_div(idx, div_cv);
  const int cg = (int)(idx - t1 * div_cv.d);
  const unsigned t2 = fast_div(t1, div_cols);
  const int oxg = (int)(t1 - t2 * div_cols.d);
  const unsigned b = fast_div(t2, div_segs);
  const int seg = (int)(t2 - b * div_segs.d);
  const int ch = cg * V;
  const int oy0 = seg * seg_rows;
  const int rows = min(seg_rows, oh - oy0);  // output rows of this segment (>= 1)
  const int ox0 = oxg * Q;

  float wt[9][V];
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) Vec<T>::load(w + tap * c + ch, wt[tap]);
  float bv[V];
#pragma unroll
  for (int v = 0; v < V; ++v) bv[v] = 0.f;
  if (bias != nullptr) {
#pragma unroll
    for (int v = 0; v < V; v += 4) {
      const float4 t = *reinterpret_cast<const float4*>(bias + ch + v);
      bv[v] = t.x; bv[v + 1] = t.y; bv[v + 2] = t.z; bv[v + 3] = t.w;
    }
  }

  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(x), 0, (int)x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(y, 0, (int)y_bytes, 0x00020000);
  const unsigned row_bytes = (unsigned)(wd * c) * ESZ;
  const unsigned img = (b * (unsigned)h) * row_bytes + (unsigned)ch * ESZ;
  const int iy_base = oy0 * S - pad;           // input row of ring position 0
  const int in_rows = (rows - 1) * S + 3;      // input rows this segment touches
  unsigned col_off[IN_COLS];
#pragma unroll
  for (int s = 0; s < IN_COLS; ++s) {
    const int ix = ox0 * S - pad + s;
    col_off[s] = (unsigned)ix < (unsigned)wd ? (unsigned)(ix * c) * ESZ : kOut;
  }
  u32x4 raw[NB][IN_COLS];
  // requests input row `r` (relative to iy_base) into ring slot `slot`
#define OGLE_DW_LOAD_ROW(slot, r)                                                               \
  {                                                                                             \
    const int iy_ = iy_base + (r);                                                              \
    const unsigned ro_ = ((r) < in_rows && (unsigned)iy_ < (unsigned)h)                         \
                             ? img + (unsigned)iy_ * row_bytes : kOut;                          \
    _Pragma("unroll") for (int s = 0; s < IN_COLS; ++s) {                                       \
      const unsigned off_ = (ro_ + col_off[s]) | ((ro_ | col_off[s]) & kOut);                   \
      raw[slot][s] = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)off_, 0, 0);                \
    }                                                                                           \
  }
#pragma unroll
  for (int j = 0; j < NB - S; ++j) OGLE_DW_LOAD_ROW(j, j);   // rows 0 .. 2 + S*(PF-1)
  const unsigned out_row_bytes = (unsigned)(ow * c) * ESZ;
  unsigned out_off = (b * (unsigned)oh + (unsigned)oy0) * out_row_bytes + (unsigned)(ox0 * c + ch) * ESZ;
  for (int t0 = 0; t0 < rows; t0 += NB) {
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int t = t0 + u;                    // output row of the segment
      if (t < rows) {
        // the S rows that output row t + PF will newly need go into the slots of the rows
        // output row t - 1 was the last to use
#pragma unroll
        for (int e = 0; e < S; ++e)
          OGLE_DW_LOAD_ROW((S * u + 3 + S * (PF - 1) + e) % NB, S * t + 3 + S * (PF - 1) + e);
        float acc[Q][V];
#pragma unroll
        for (int q = 0; q < Q; ++q)
#pragma unroll
          for (int v = 0; v < V; ++v) acc[q][v] = bv[v];
#pragma unroll
        for (int ky = 0; ky < 3; ++ky) {
          float in[IN_COLS][V];
#pragma unroll
          for (int s = 0; s < IN_COLS; ++s) Vec<T>::unpack(raw[(S * u + ky) % NB][s], in[s]);
#pragma unroll
          for (int q = 0; q < Q; ++q)
#pragma unroll
            for (int kx = 0; kx < 3; ++kx)
#pragma unroll
              for (int v = 0; v < V; ++v) acc[q][v] += wt[ky * 3 + kx][v] * in[q * S + kx][v];
        }
#pragma unroll
        for (int q = 0; q < Q; ++q) {
          float out[V];
#pragma unroll
          for (int v = 0; v < V; ++v) out[v] = apply_epilogue(acc[q][v], ep);
          const unsigned off = ox0 + q < ow ? out_off + (unsigned)(q * c) * ESZ : kOut;
          __builtin_amdgcn_raw_buffer_store_b128(Vec<T>::pack(out), ry, (int)off, 0, kResultStoreAux);
        }
        out_off += out_row_bytes;
      }
    }
  }
#undef OGLE_DW_LOAD_ROW
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

template <typename T, int S, int Q, int PF>
int32_t launch_rows(const OgleConvArgs& a, hipStream_t s, const Epilogue& ep, int seg_rows) {
  constexpr int V = Vec<T>::N;
  const int segs = (a.out_h + seg_rows - 1) / seg_rows, cols = (a.out_w + Q - 1) / Q, cv = a.in_c / V;
  const long total = (long)a.n * segs * cols * cv;
  const int blocks = (ceil_div(total, 256) + 7) / 8 * 8;  // whole XCD rounds
  launch((dwconv3x3_rows<T, S, Q, PF>), dim3(blocks), dim3(256), 0, s,
                     static_cast<const T*>(a.input_dev), static_cast<const T*>(a.filter_dev),
                     a.bias_dev, static_cast<T*>(a.output_dev), a.in_h, a.in_w, a.in_c, a.out_h,
                     a.out_w, a.padding, ep,
                     (unsigned)((long)a.n * a.in_h * a.in_w * a.in_c * sizeof(T)),
                     (unsigned)((long)a.n * a.out_h * a.out_w * a.in_c * sizeof(T)), (unsigned)total,
                     make_fast_div((unsigned)cv), make_fast_div((unsigned)cols),
                     make_fast_div((unsigned)segs), seg_rows);
  return check_launch("dwconv3x3_rows");
}

// Segment length and columns per thread, measured on MI355X over the MobileNet shapes
// (batch 16; 150x150x32 ... 10x10x1024): two columns per thread at stride 1 (input
// requests per output: 2), one at stride 2 (two columns would need five input columns in
// registers); one step of prefetch (two gained nothing); segments of 13 rows on the large
// maps (halo rows re-read by the next segment: 2 in 15) and of 4 rows on maps of 38 rows
// and below, where the number of waves, not the re-read rows, decides the time.
template <typename T, int S>
int32_t pick_rows(const OgleConvArgs& a, hipStream_t s, const Epilogue& ep) {
  int seg_rows = (S == 1 && a.out_h > 40) ? 13 : 4;
  // Few images: with fewer than one workgroup per compute unit the launch is a handful of
  // long serial walks (150x150x32 at batch 1: 28 workgroups of 13-row walks, 7.6 us); shorter
  // segments make more of them (the rows a segment re-reads do not matter at this size).
  {
    constexpr int V = Vec<T>::N;
    const int q = (S == 1 && a.out_w >= 2) ? 2 : 1;
    auto workgroups = [&](int rows) {
      return ((long)a.n * ((a.out_h + rows - 1) / rows) * ((a.out_w + q - 1) / q) * (a.in_c / V) + 255) / 256;
    };
    while (seg_rows > 2 && workgroups(seg_rows) < 256) seg_rows = seg_rows > 4 ? 4 : 2;
  }
  if (S == 1 && a.out_w >= 2) return launch_rows<T, S, 2, 1>(a, s, ep, seg_rows);
  return launch_rows<T, S, 1, 1>(a, s, ep, seg_rows);
}

template <typename T>
int32_t run_dw(const OgleConvArgs& a, hipStream_t s) {
  const Epilogue ep = make_epilogue(a.act, a.min_value, a.max_value, a.act_variant);
  constexpr int V = Vec<T>::N;
  // the 3x3 kernel addresses the input with 32-bit byte offsets (buffer loads)
  // and the bias with 16-byte loads
  const bool fits = (long)a.n * a.in_h * a.in_w * a.in_c * (long)sizeof(T) < 0x7fffffffL &&
                    (long)a.n * a.out_h * a.out_w * a.in_c * (long)sizeof(T) < 0x7fffffffL &&
                    (reinterpret_cast<uintptr_t>(a.bias_dev) & 15u) == 0;
  if (a.kernel_size == 3 && a.dilation == 1 && a.in_c % V == 0 && fits &&
      (a.stride == 1 || a.stride == 2)) {
    if (a.stride == 1) return pick_rows<T, 1>(a, s, ep);
    return pick_rows<T, 2>(a, s, ep);
  }
  const long total = (long)a.n * a.out_h * a.out_w * a.out_c;
  int blocks = ceil_div(total, 256);
  if (blocks > 256 * 64) blocks = 256 * 64;
  if (blocks < 1) blocks = 1;
  launch((dwconv_general<T>), dim3(blocks), dim3(256), 0, s,
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
