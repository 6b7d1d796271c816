// Direct convolution over NHWC: the general path (any kernel size, stride,
// padding, dilation, group count and channel count).  The MFMA implicit-GEMM
// kernel takes the shapes it is eligible for; everything else lands here:
// small input-channel counts (the RGB stem), channel counts that are not a
// multiple of 4, grouped convolutions with 1 < group < C.
//
// Semantics follow conv2d.glsl:29-92 / conv2d_grp.glsl:30-123: accumulator
// starts at the bias, taps outside the image are skipped, then the fused
// activation.  Accumulation order is ky, kx, input channel ascending.
#include <algorithm>
#include <type_traits>
#include "common.h"

namespace ogle {
namespace {

// Small-K kernel (the RGB stem): one thread produces OPT consecutive output
// channels of one pixel.  Filter taps [O][K] (K = k*k*C, OHWI order) are staged
// through LDS transposed to [K][O]; a wave then reads the OPT weights of one
// (tap, channel) as 16-byte broadcasts, and each input value is loaded once per
// thread.  O must be a multiple of OPT.
template <typename T, int OPT>
__global__ __launch_bounds__(256) void conv_direct_small_k(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ y, int n, int h, int wd, int c, int oh, int ow, int o, int k, int stride,
    int pad, int dil, Epilogue ep, int ktot) {
  extern __shared__ __attribute__((aligned(16))) float lds_w[];  // [ktot][o]
  for (int i = threadIdx.x; i < ktot * o; i += blockDim.x) {
    int oc = i / ktot, kk = i - oc * ktot;
    lds_w[kk * o + oc] = to_f32(w[i]);
  }
  __syncthreads();
  const int groups_per_pixel = o / OPT;
  const long total = (long)n * oh * ow * groups_per_pixel;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int og = (int)(idx % groups_per_pixel);
    long pix = idx / groups_per_pixel;
    const int ox = (int)(pix % ow);
    pix /= ow;
    const int oy = (int)(pix % oh);
    const int b = (int)(pix / oh);
    const int oc0 = og * OPT;
    float acc[OPT];
#pragma unroll
    for (int j = 0; j < OPT; ++j) acc[j] = bias != nullptr ? bias[oc0 + j] : 0.f;
    for (int r = 0; r < k; ++r) {
      const int iy = oy * stride - pad + r * dil;
      if (iy < 0 || iy >= h) continue;
      for (int s = 0; s < k; ++s) {
        const int ix = ox * stride - pad + s * dil;
        if (ix < 0 || ix >= wd) continue;
        const T* xp = x + (((long)b * h + iy) * wd + ix) * c;
        const float* wp = lds_w + (long)((r * k + s) * c) * o + oc0;
        for (int ci = 0; ci < c; ++ci) {
          const float xv = to_f32(xp[ci]);
          const float4* w4 = reinterpret_cast<const float4*>(wp + ci * o);
#pragma unroll
          for (int j = 0; j < OPT / 4; ++j) {
            const float4 wv = w4[j];
            acc[4 * j + 0] += xv * wv.x;
            acc[4 * j + 1] += xv * wv.y;
            acc[4 * j + 2] += xv * wv.z;
            acc[4 * j + 3] += xv * wv.w;
          }
        }
      }
    }
    T* yp = y + (((long)b * oh + oy) * ow + ox) * o + oc0;
    if constexpr (sizeof(T) == 4) {
#pragma unroll
      for (int j = 0; j < OPT / 4; ++j)
        reinterpret_cast<float4*>(yp)[j] =
            make_float4(apply_epilogue(acc[4 * j], ep), apply_epilogue(acc[4 * j + 1], ep),
                        apply_epilogue(acc[4 * j + 2], ep), apply_epilogue(acc[4 * j + 3], ep));
    } else {
#pragma unroll
      for (int j = 0; j < OPT; ++j) yp[j] = from_f32<T>(apply_epilogue(acc[j], ep));
    }
  }
}

// Stem kernel: few input channels, K = k*k*C <= 32 (the RGB stem has K = 27), on
// the MFMA units.  A wave owns 32 output pixels x 32 output channels at a time and
// contracts K with KS = ceil(K/2) v_mfma_f32_32x32x2_f32: lane l supplies
// A[pixel l%32][k = 2s + l/32] and B[k][channel l%32].  The filter values a lane
// needs (KS of them) are loaded once and stay in registers while the wave walks
// over pixel tiles; the lane's KS input taps are gathered straight from global
// memory (the whole receptive field of a tile is a few KB and is served by the
// vector cache), all loads of a tile in flight before the first MFMA.  Rows past
// the end, taps outside the image and the odd K tail contribute zeros.
typedef float stem_acc_t __attribute__((ext_vector_type(16)));
typedef unsigned int stem_u32x2 __attribute__((ext_vector_type(2)));

// 32-bit element offset that no operand reaches (they are kept below 2^31 bytes):
// a buffer access at it reads zero / is dropped.
constexpr unsigned kStemOutOfRange = 0x80000000u;

template <typename T>
__device__ __forceinline__ float stem_load(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0));
  } else {
    const unsigned short v = __builtin_amdgcn_raw_buffer_load_b16(r, (int)byte_off, 0, 0);
    return __half2float(__builtin_bit_cast(__half, v));
  }
}
template <typename T>
__device__ __forceinline__ void stem_store(__amdgpu_buffer_rsrc_t r, unsigned byte_off, float v) {
  if constexpr (sizeof(T) == 4) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, (int)byte_off, 0, kResultStoreAux);
  } else {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, __float2half_rn(v)), r,
                                          (int)byte_off, 0, kResultStoreAux);
  }
}

// What K index kidx means, worked out on the host: the tap's (dy, dx) relative to
// the pixel's top-left input position and its element offset from there.
struct StemTaps {
  int dy[32], dx[32], off[32];
};

template <typename T, int KS>
__global__ __launch_bounds__(256) void conv_stem_mfma(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ y, int h, int wd, int c, int oh, int ow, int o, int stride, Epilogue ep,
    int ktot, int m_total, int tiles_m, unsigned x_bytes, unsigned y_bytes, StemTaps taps) {
  constexpr unsigned ESZ = sizeof(T);
  const int lane = threadIdx.x & 63;
  const int l32 = lane & 31, lh = lane >> 5;
  const int wave = (int)(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int waves = (int)(gridDim.x * 4);
  const __amdgpu_buffer_rsrc_t rx =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x), 0, (int)x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(y, 0, (int)y_bytes, 0x00020000);
  // this lane's K indices: kidx = 2s + lane/32 (entries past K never fall inside the image)
  int tap_dy[KS], tap_dx[KS], tap_off[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    tap_dy[s] = lh ? taps.dy[2 * s + 1] : taps.dy[2 * s];
    tap_dx[s] = lh ? taps.dx[2 * s + 1] : taps.dx[2 * s];
    tap_off[s] = lh ? taps.off[2 * s + 1] : taps.off[2 * s];
  }
  for (int n0 = 0; n0 < o; n0 += 32) {
    const int col = n0 + l32;
    float bval[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int kidx = 2 * s + lh;
      bval[s] = (col < o && kidx < ktot) ? to_f32(w[(long)col * ktot + kidx]) : 0.f;
    }
    const float bias_v = (bias != nullptr && col < o) ? bias[col] : 0.f;
    // the taps of a tile, all issued at once; a tile past the end reads zeros without touching memory
    auto gather = [&](int tile, float (&dst)[KS]) {
      const int m = tile * 32 + l32;
      const int ox = m % ow;
      const int t = m / ow;
      const int oy = t % oh;
      const int b = t / oh;
      const int iy0 = oy * stride, ix0 = ox * stride;
      const int base = (tile < tiles_m && m < m_total) ? ((b * h + iy0) * wd + ix0) * c : -0x40000000;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const bool in = (unsigned)(iy0 + tap_dy[s]) < (unsigned)h &&
                        (unsigned)(ix0 + tap_dx[s]) < (unsigned)wd && base >= 0;
        dst[s] = stem_load<T>(rx, in ? (unsigned)(base + tap_off[s]) * ESZ : kStemOutOfRange);
      }
    };
    float a[KS], a_next[KS];
    gather(wave, a);
    for (int tile = wave; tile < tiles_m; tile += waves) {
      // the next tile's taps are in flight while this tile is multiplied and stored
      gather(tile + waves, a_next);
      stem_acc_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], bval[s], acc, 0, 0, 0);
#pragma unroll
      for (int s = 0; s < KS; ++s) a[s] = a_next[s];
      // register r of lane l: pixel 8*(r/4) + 4*(l/32) + r%4 of the tile, channel l%32
      const int row0 = tile * 32 + lh * 4;
      const unsigned off0 = (unsigned)(row0 * o + col);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int dr = (r >> 2) * 8 + (r & 3);
        const bool ok = row0 + dr < m_total && col < o;
        stem_store<T>(ry, ok ? (off0 + (unsigned)(dr * o)) * ESZ : kStemOutOfRange,
                      apply_epilogue(acc[r] + bias_v, ep));
      }
    }
  }
}

// The RGB stem (3x3 taps on 3 channels, fp32, even stride, padding 1, even width, output
// channels a multiple of 32): the nine values one filter row needs for a pixel are nine
// consecutive floats of an input row, so instead of 27 scalar gathers (a counter run showed 32
// vector-cache accesses per such load instruction and the kernel bound by them) a lane fetches
// its share of K as runs of 8-byte pairs.  With an even stride and padding 1 a pixel's run starts
// at an odd float of its row, so the pair that starts one float earlier is 8-byte aligned.  The
// lower half of the wave takes filter row 0 and the first five values of row 1, the upper half
// the last four values of row 1 (plus one zero) and row 2: five pairs for the 9-run and three
// for the rest, eight load instructions instead of fourteen, each twice as wide.  The
// contraction order is permuted to match (the filter values a lane keeps are picked
// accordingly).  Values that fall into padding columns are cleared with a per-lane test, and
// so are padding rows, rows past the end and pairs outside the tensor.
template <int UNUSED = 0>
__global__ __launch_bounds__(256) void conv_stem_rgb_mfma(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
    float* __restrict__ y, int h, int wd, int oh, int ow, int o, int stride, Epilogue ep,
    int m_total, int tiles_m, unsigned x_bytes, unsigned y_bytes) {
  constexpr int KS = 14;
  const int lane = threadIdx.x & 63;
  const int l32 = lane & 31, lh = lane >> 5;
  const int wave = (int)(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int waves = (int)(gridDim.x * 4);
  const __amdgpu_buffer_rsrc_t rx =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x), 0, (int)x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(y, 0, (int)y_bytes, 0x00020000);
  const int row_floats = wd * 3;
  const unsigned total_floats = x_bytes / 4u;
  const int run0_ky = lh ? 2 : 0;
  const int run1_count = lh ? 4 : 5;
  for (int n0 = 0; n0 < o; n0 += 32) {
    const int col = n0 + l32;
    float bval[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int k = s < 9 ? run0_ky * 9 + s : 9 + (lh ? 5 : 0) + (s - 9);
      bval[s] = (s < 9 || s - 9 < run1_count) ? w[(long)col * 27 + k] : 0.f;
    }
    const float bias_v = bias != nullptr ? bias[col] : 0.f;
    for (int tile = wave; tile < tiles_m; tile += waves) {
      const int m = tile * 32 + l32;
      const int ox = m % ow;
      const int t = m / ow;
      const int oy = t % oh;
      const int b = t / oh;
      const int iy0 = oy * stride - 1;
      const int f0 = (ox * stride - 1) * 3;  // first float of a pixel's 9-run within an input row (odd)
      // PAIRS 8-byte pairs of input row iy from float f (even) on.  Plain 8-byte loads (the
      // 8-byte buffer load builtin compiles to a one-dword load with this toolchain); a pair
      // outside the tensor, or of a row that does not exist, is read from the tensor's start
      // instead and its values are cleared.
      auto fetch = [&](int iy, int f, float* v, auto pairs) {
        const bool row_ok = m < m_total && (unsigned)iy < (unsigned)h;
        const int first = (b * h + iy) * row_floats + f;  // may be negative in the first row
#pragma unroll
        for (int i = 0; i < decltype(pairs)::value; ++i) {
          const int at = first + 2 * i;
          const bool ok = row_ok && (unsigned)at + 1u < total_floats;
          const unsigned byte_off = ok ? (unsigned)at * 4u : 0u;
          const float2 q = *reinterpret_cast<const float2*>(reinterpret_cast<const char*>(x) + byte_off);
          v[2 * i] = ok ? q.x : 0.f;
          v[2 * i + 1] = ok ? q.y : 0.f;
        }
      };
      float v0[10], v1[6];
      fetch(iy0 + run0_ky, f0 - 1, v0, std::integral_constant<int, 5>());
      // filter row 1: floats [f0, f0 + 5) for the lower half, [f0 + 5, f0 + 9) for the upper
      const int f1 = lh ? f0 + 5 : f0 - 1;
      fetch(iy0 + 1, f1, v1, std::integral_constant<int, 3>());
      float a[KS];
#pragma unroll
      for (int j = 0; j < 9; ++j)
        a[j] = (unsigned)(f0 + j) < (unsigned)row_floats ? v0[j + 1] : 0.f;
#pragma unroll
      for (int j = 0; j < 5; ++j) {
        const int f = lh ? f0 + 5 + j : f0 + j;
        const float val = lh ? v1[j] : v1[j + 1];
        a[9 + j] = ((unsigned)f < (unsigned)row_floats && j < run1_count) ? val : 0.f;
      }
      stem_acc_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], bval[s], acc, 0, 0, 0);
      // register r of lane l: pixel 8*(r/4) + 4*(l/32) + r%4 of the tile, channel l%32; rows
      // past the end lie past the end of the buffer and are dropped by the range check
      const unsigned off0 = (unsigned)((tile * 32 + lh * 4) * o + col) * 4u;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int dr = (r >> 2) * 8 + (r & 3);
        __builtin_amdgcn_raw_buffer_store_b32(
            __builtin_bit_cast(unsigned, apply_epilogue(acc[r] + bias_v, ep)), ry,
            (int)(off0 + (unsigned)(dr * o) * 4u), 0, kResultStoreAux);
      }
    }
  }
}

// Fully general kernel: one thread per output element, output channel
// fastest.  Filter OHWI with I = c/groups.
template <typename T>
__global__ __launch_bounds__(256) void conv_direct_general(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ y, int n, int h, int wd, int c, int oh, int ow, int o, int k, int stride,
    int pad, int dil, int groups, Epilogue ep) {
  const int cpg = c / groups;
  const int opg = o / groups;
  const long total = (long)n * oh * ow * o;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int oc = (int)(idx % o);
    long pix = idx / o;
    const int ox = (int)(pix % ow);
    pix /= ow;
    const int oy = (int)(pix % oh);
    const int b = (int)(pix / oh);
    const int g = oc / opg;
    float acc = bias != nullptr ? bias[oc] : 0.f;
    const T* wf = w + (long)oc * k * k * cpg;
    for (int r = 0; r < k; ++r) {
      const int iy = oy * stride - pad + r * dil;
      if (iy < 0 || iy >= h) continue;
      for (int s = 0; s < k; ++s) {
        const int ix = ox * stride - pad + s * dil;
        if (ix < 0 || ix >= wd) continue;
        const T* xp = x + (((long)b * h + iy) * wd + ix) * c + g * cpg;
        const T* wp = wf + (r * k + s) * cpg;
        for (int ci = 0; ci < cpg; ++ci) acc += to_f32(xp[ci]) * to_f32(wp[ci]);
      }
    }
    y[idx] = from_f32<T>(apply_epilogue(acc, ep));
  }
}

template <typename T>
int32_t run_direct(const OgleConvArgs& a, hipStream_t s) {
  const Epilogue ep = make_epilogue(a.act, a.min_value, a.max_value, a.act_variant);
  const T* x = static_cast<const T*>(a.input_dev);
  const T* w = static_cast<const T*>(a.filter_dev);
  T* y = static_cast<T*>(a.output_dev);
  const int ktot = a.kernel_size * a.kernel_size * a.in_c;
  const size_t lds = sizeof(float) * (size_t)ktot * a.out_c;
  const long pixels_all = (long)a.n * a.out_h * a.out_w;
  const long esz = (long)sizeof(T);
  const long x_bytes = (long)a.n * a.in_h * a.in_w * a.in_c * esz;
  const long y_bytes = pixels_all * a.out_c * esz;
  if (a.group == 1 && ktot <= 32 && pixels_all >= 4096 && x_bytes < 0x7fffffffL &&
      y_bytes < 0x7fffffffL) {
    const int tiles_m = (int)((pixels_all + 31) / 32);
    // a wave keeps its filter values while it walks over tiles: one wave per tile
    // until every compute unit has three workgroups (measured best), then more tiles
    // per wave
    int blocks = (tiles_m + 3) / 4;
    if (blocks > 256 * 3) blocks = 256 * 3;
    const int ks = (ktot + 1) / 2;
    StemTaps taps;
    for (int kidx = 0; kidx < 32; ++kidx) {
      const int tap = kidx / a.in_c, ci = kidx % a.in_c;
      taps.dy[kidx] = (tap / a.kernel_size) * a.dilation - a.padding;
      taps.dx[kidx] = (tap % a.kernel_size) * a.dilation - a.padding;
      taps.off[kidx] = (taps.dy[kidx] * a.in_w + taps.dx[kidx]) * a.in_c + ci;
      if (kidx >= ktot) taps.dy[kidx] = -0x40000000;
    }
    if (sizeof(T) == 4 && a.kernel_size == 3 && a.in_c == 3 && a.dilation == 1 && a.padding == 1 &&
        a.stride % 2 == 0 && a.in_w % 2 == 0 && a.out_c % 32 == 0 &&
        reinterpret_cast<uintptr_t>(x) % 8 == 0) {
      // four workgroups per compute unit measured best for this one (17.3 against 18.3 us at batch 16)
      const int rgb_blocks = std::min((tiles_m + 3) / 4, 256 * 4);
      launch((conv_stem_rgb_mfma<0>), dim3(rgb_blocks), dim3(256), 0, s,
             reinterpret_cast<const float*>(x), reinterpret_cast<const float*>(w), a.bias_dev,
             reinterpret_cast<float*>(y), a.in_h, a.in_w, a.out_h, a.out_w, a.out_c, a.stride, ep,
             (int)pixels_all, tiles_m, (unsigned)x_bytes, (unsigned)y_bytes);
      return check_launch("conv_stem_rgb_mfma");
    }
#define OGLE_STEM_CASE(KS)                                                                        \
  launch((conv_stem_mfma<T, KS>), dim3(blocks), dim3(256), 0, s, x, w, a.bias_dev, y,  \
                     a.in_h, a.in_w, a.in_c, a.out_h, a.out_w, a.out_c, a.stride, ep, ktot,       \
                     (int)pixels_all, tiles_m, (unsigned)x_bytes, (unsigned)y_bytes, taps)
    if (ks <= 5) OGLE_STEM_CASE(5);
    else if (ks <= 9) OGLE_STEM_CASE(9);
    else if (ks <= 14) OGLE_STEM_CASE(14);
    else OGLE_STEM_CASE(16);
#undef OGLE_STEM_CASE
    return check_launch("conv_stem_mfma");
  }
  if (a.group == 1 && lds <= 48 * 1024 && a.out_c % 4 == 0) {
    // 16 channels per thread when that still leaves enough threads to fill the chip
    const long pixels = (long)a.n * a.out_h * a.out_w;
    const bool wide = a.out_c % 16 == 0 && pixels * (a.out_c / 16) >= 256L * 256 * 4;
    const int opt = wide ? 16 : 4;
    const long total = pixels * (a.out_c / opt);
    int blocks = ceil_div(total, 256);
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (blocks < 1) blocks = 1;
    if (wide) {
      launch((conv_direct_small_k<T, 16>), dim3(blocks), dim3(256), lds, s, x, w,
                         a.bias_dev, y, a.n, a.in_h, a.in_w, a.in_c, a.out_h, a.out_w, a.out_c,
                         a.kernel_size, a.stride, a.padding, a.dilation, ep, ktot);
    } else {
      launch((conv_direct_small_k<T, 4>), dim3(blocks), dim3(256), lds, s, x, w,
                         a.bias_dev, y, a.n, a.in_h, a.in_w, a.in_c, a.out_h, a.out_w, a.out_c,
                         a.kernel_size, a.stride, a.padding, a.dilation, ep, ktot);
    }
    return check_launch("conv_direct_small_k");
  }
  const long total = (long)a.n * a.out_h * a.out_w * a.out_c;
  int blocks = ceil_div(total, 256);
  if (blocks > 256 * 64) blocks = 256 * 64;
  if (blocks < 1) blocks = 1;
  launch((conv_direct_general<T>), dim3(blocks), dim3(256), 0, s, x, w, a.bias_dev,
                     y, a.n, a.in_h, a.in_w, a.in_c, a.out_h, a.out_w, a.out_c, a.kernel_size,
                     a.stride, a.padding, a.dilation, a.group, ep);
  return check_launch("conv_direct_general");
}

}  // namespace

int32_t launch_conv_direct(const OgleConvArgs& a, hipStream_t s) {
  if (a.dtype == OGLE_F16) return run_direct<__half>(a, s);
  return run_direct<float>(a, s);
}

}  // namespace ogle
