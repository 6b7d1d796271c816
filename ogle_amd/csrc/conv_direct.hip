// Direct convolution over NHWC: the general path (any kernel size, stride,
// padding, dilation, group count and channel count).  The MFMA implicit-GEMM
// kernel takes the shapes it is eligible for; everything else lands here:
// small input-channel counts (the RGB stem), channel counts that are not a
// multiple of 4, grouped convolutions with 1 < group < C.
//
// Semantics follow conv2d.glsl:29-92 / conv2d_grp.glsl:30-123: accumulator
// starts at the bias, taps outside the image are skipped, then the fused
// activation.  Accumulation order is ky, kx, input channel ascending.
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
      hipLaunchKernelGGL((conv_direct_small_k<T, 16>), dim3(blocks), dim3(256), lds, s, x, w,
                         a.bias_dev, y, a.n, a.in_h, a.in_w, a.in_c, a.out_h, a.out_w, a.out_c,
                         a.kernel_size, a.stride, a.padding, a.dilation, ep, ktot);
    } else {
      hipLaunchKernelGGL((conv_direct_small_k<T, 4>), dim3(blocks), dim3(256), lds, s, x, w,
                         a.bias_dev, y, a.n, a.in_h, a.in_w, a.in_c, a.out_h, a.out_w, a.out_c,
                         a.kernel_size, a.stride, a.padding, a.dilation, ep, ktot);
    }
    return check_launch("conv_direct_small_k");
  }
  const long total = (long)a.n * a.out_h * a.out_w * a.out_c;
  int blocks = ceil_div(total, 256);
  if (blocks > 256 * 64) blocks = 256 * 64;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((conv_direct_general<T>), dim3(blocks), dim3(256), 0, s, x, w, a.bias_dev,
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
