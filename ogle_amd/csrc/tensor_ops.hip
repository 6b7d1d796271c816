// Bandwidth-bound tensor kernels that share the conv path's NHWC buffers:
// pooling (pool.glsl), concatenation (concat_multi.glsl), the filter repack that
// replaces the NCHW -> HWN4C4 upload shader, and element-type conversion.
#include "common.h"

namespace ogle {
namespace {

// ---------------------------------------------------------------- pooling --
// One thread per output element group; channels fastest so that a wave reads and
// writes contiguous NHWC runs.  Semantics of pool.glsl:19-66: max takes the
// first in-image tap then max of the rest (no in-image tap -> 0); average sums
// in-image taps and always divides by k*k.  Tap order kx outer, ky inner.
template <typename T, int V>
__global__ __launch_bounds__(256) void pool_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                   int n, int h, int wd, int c, int oh, int ow,
                                                   int k, int stride, int pad, int pool_type) {
  const int cv = c / V;
  const long total = (long)n * oh * ow * cv;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int cg = (int)(idx % cv);
    long pix = idx / cv;
    const int ox = (int)(pix % ow);
    pix /= ow;
    const int oy = (int)(pix % oh);
    const int b = (int)(pix / oh);
    float v[V];
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = 0.f;
    bool first = true;
    for (int i = 0; i < k; ++i) {
      const int ix = ox * stride + i - pad;
      if (ix < 0 || ix >= wd) continue;
      for (int jy = 0; jy < k; ++jy) {
        const int iy = oy * stride + jy - pad;
        if (iy < 0 || iy >= h) continue;
        const T* p = x + (((long)b * h + iy) * wd + ix) * c + cg * V;
        float item[V];
        if constexpr (V == 4 && sizeof(T) == 4) {
          const float4 t = *reinterpret_cast<const float4*>(p);
          item[0] = t.x; item[1] = t.y; item[2] = t.z; item[3] = t.w;
        } else {
#pragma unroll
          for (int j = 0; j < V; ++j) item[j] = to_f32(p[j]);
        }
        if (pool_type == OGLE_POOL_MAX) {
          if (first) {
#pragma unroll
            for (int j = 0; j < V; ++j) v[j] = item[j];
            first = false;
          } else {
#pragma unroll
            for (int j = 0; j < V; ++j) v[j] = v[j] > item[j] ? v[j] : item[j];
          }
        } else {
#pragma unroll
          for (int j = 0; j < V; ++j) v[j] += item[j];
        }
      }
    }
    if (pool_type != OGLE_POOL_MAX) {
      const float denom = (float)(k * k);
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = v[j] / denom;
    }
    T* q = y + (((long)b * oh + oy) * ow + ox) * c + cg * V;
    if constexpr (V == 4 && sizeof(T) == 4) {
      store_result16(q, make_float4(v[0], v[1], v[2], v[3]));
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) q[j] = from_f32<T>(v[j]);
    }
  }
}

// Unsigned division by a number fixed at launch, exact below 2^31.
struct PoolDiv {
  unsigned mul, shift, d;
};
__device__ __forceinline__ unsigned pool_div(unsigned n, const PoolDiv& f) {
  return (__umulhi(n, f.mul) + n) >> f.shift;
}
PoolDiv make_pool_div(unsigned d) {
  PoolDiv f{0, 0, d};
  unsigned l = 0;
  while ((1ull << l) < d) ++l;
  f.shift = l;
  f.mul = (unsigned)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
  return f;
}

// Small windows (K = 2, 3), fp32, channel count a multiple of 4: one thread per
// 16-byte channel vector of one output pixel; the K*K taps are branch-free buffer
// loads, all in flight before the first comparison (a tap outside the image gets an
// out-of-range offset; its lanes are then masked out of the maximum, or add the zeros
// they read to the average).  Same results as pool_kernel.
template <int K>
__global__ __launch_bounds__(256) void pool_small_kernel(
    const float* __restrict__ x, float* __restrict__ y, int h, int wd, int c, int oh, int ow,
    int stride, int pad, int pool_type, unsigned total, unsigned x_bytes, unsigned y_bytes,
    PoolDiv div_cv, PoolDiv div_ow, PoolDiv div_oh) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  constexpr unsigned kOut = 0x80000000u;
  // consecutive workgroups (neighbouring output rows, whose windows share input rows)
  // are kept on one XCD so that the re-read rows hit that XCD's L2
  const unsigned idx = (unsigned)xcd_swizzle((int)blockIdx.x, (int)gridDim.x) * 256u + threadIdx.x;
  if (idx >= total) return;
  const unsigned t1 = pool_div(idx, div_cv);
  const unsigned cg = idx - t1 * div_cv.d;
  const unsigned t2 = pool_div(t1, div_ow);
  const int ox = (int)(t1 - t2 * div_ow.d);
  const unsigned b = pool_div(t2, div_oh);
  const int oy = (int)(t2 - b * div_oh.d);
  const __amdgpu_buffer_rsrc_t rx =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x), 0, (int)x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(y, 0, (int)y_bytes, 0x00020000);
  const unsigned row_bytes = (unsigned)(wd * c) * 4u;
  const unsigned img = b * (unsigned)h * row_bytes + cg * 16u;
  unsigned row_off[K], col_off[K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int iy = oy * stride + j - pad;
    row_off[j] = (unsigned)iy < (unsigned)h ? img + (unsigned)iy * row_bytes : kOut;
    const int ix = ox * stride + j - pad;
    col_off[j] = (unsigned)ix < (unsigned)wd ? (unsigned)(ix * c) * 4u : kOut;
  }
  u32x4 raw[K][K];  // [kx][ky], the shader's tap order
#pragma unroll
  for (int i = 0; i < K; ++i)
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const unsigned off = (row_off[j] + col_off[i]) | ((row_off[j] | col_off[i]) & kOut);
      raw[i][j] = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)off, 0, 0);
    }
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (pool_type == OGLE_POOL_MAX) {
    bool any = false;
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
      for (int j = 0; j < K; ++j) {
        const bool ok = ((row_off[j] | col_off[i]) & kOut) == 0;
        const float item[4] = {__uint_as_float(raw[i][j].x), __uint_as_float(raw[i][j].y),
                               __uint_as_float(raw[i][j].z), __uint_as_float(raw[i][j].w)};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          // the first in-image tap initialises, later ones take the maximum (pool.glsl:48-55)
          const float m = v[q] > item[q] ? v[q] : item[q];
          v[q] = ok ? (any ? m : item[q]) : v[q];
        }
        any = any || ok;
      }
  } else {
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
      for (int j = 0; j < K; ++j) {
        v[0] += __uint_as_float(raw[i][j].x);
        v[1] += __uint_as_float(raw[i][j].y);
        v[2] += __uint_as_float(raw[i][j].z);
        v[3] += __uint_as_float(raw[i][j].w);
      }
    const float denom = (float)(K * K);
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] = v[q] / denom;
  }
  u32x4 out;
  out.x = __float_as_uint(v[0]); out.y = __float_as_uint(v[1]);
  out.z = __float_as_uint(v[2]); out.w = __float_as_uint(v[3]);
  const unsigned off = ((b * (unsigned)oh + (unsigned)oy) * (unsigned)ow + (unsigned)ox) *
                           (unsigned)c * 4u + cg * 16u;
  __builtin_amdgcn_raw_buffer_store_b128(out, ry, (int)off, 0, kResultStoreAux);
}

// Global average pooling with large windows: one workgroup per (image, 64
// channel slab): lanes stride over pixels, partial sums reduced through LDS.
// The summation order differs from the shader's sequential one; the result
// agrees within fp32 rounding of the window sum.
template <typename T>
__global__ __launch_bounds__(256) void global_avg_kernel(const T* __restrict__ x,
                                                         T* __restrict__ y, int hw, int c) {
  __shared__ float part[4][64];
  const int b = blockIdx.y;
  const int ch = blockIdx.x * 64 + (threadIdx.x & 63);
  const int w = threadIdx.x >> 6;
  float s = 0.f;
  if (ch < c)
    for (int p = w; p < hw; p += 4) s += to_f32(x[((long)b * hw + p) * c + ch]);
  part[w][threadIdx.x & 63] = s;
  __syncthreads();
  if (w == 0 && ch < c) {
    s = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
    y[(long)b * c + ch] = from_f32<T>(s / (float)hw);
  }
}

// ----------------------------------------------------------------- concat --
struct ConcatPlan {
  const void* in[OGLE_CONCAT_MAX_INPUTS];
  long run[OGLE_CONCAT_MAX_INPUTS];    // elements (or vectors) per outer step of input i
  long start[OGLE_CONCAT_MAX_INPUTS];  // offset of input i within an output outer step
  long out_run;                        // elements (or vectors) per outer step of the output
  long total;                          // outer * out_run
  int n;
};

// One launch copies every input into its slice: the output is enumerated once,
// each element (or 16-byte vector) finds its source by its position inside the
// output's outer step.  Loads and stores are contiguous within a run.
template <typename E>
__global__ __launch_bounds__(256) void concat_kernel(ConcatPlan p, E* __restrict__ out) {
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < p.total;
       idx += (long)gridDim.x * blockDim.x) {
    const long ob = idx / p.out_run;
    const long rem = idx - ob * p.out_run;
    int i = 0;
#pragma unroll 1
    for (int j = 1; j < p.n; ++j)
      if (rem >= p.start[j]) i = j;
    const E* src = static_cast<const E*>(p.in[i]);
    out[idx] = src[ob * p.run[i] + (rem - p.start[i])];
  }
}

// -------------------------------------------------------------- transpose --
struct TransposePlan {
  int out_shape[4];
  long in_stride[4];  // input stride (elements) of output dimension d
  long total;
};

// One thread per output element, output order; an identity permutation is a copy
// and is done with 16-byte vectors by the launcher instead.
template <typename E>
__global__ __launch_bounds__(256) void transpose_kernel(TransposePlan p, const E* __restrict__ in,
                                                        E* __restrict__ out) {
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < p.total;
       idx += (long)gridDim.x * blockDim.x) {
    long t = idx;
    const int d3 = (int)(t % p.out_shape[3]); t /= p.out_shape[3];
    const int d2 = (int)(t % p.out_shape[2]); t /= p.out_shape[2];
    const int d1 = (int)(t % p.out_shape[1]); t /= p.out_shape[1];
    const int d0 = (int)t;
    out[idx] = in[d0 * p.in_stride[0] + d1 * p.in_stride[1] + d2 * p.in_stride[2] +
                  d3 * p.in_stride[3]];
  }
}

// ------------------------------------------------------------ filter pack --
// OIHW fp32 -> OHWI (layout 0) or [kh*kw][O] for depthwise (layout 1, I == 1).
template <typename T>
__global__ __launch_bounds__(256) void pack_filter_kernel(const float* __restrict__ src,
                                                          T* __restrict__ dst, int layout, int o,
                                                          int ci, int kh, int kw) {
  const long total = (long)o * ci * kh * kw;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    // idx enumerates the destination
    long s;
    if (layout == OGLE_FILTER_OHWI) {
      const int i = (int)(idx % ci);
      long t = idx / ci;
      const int kx = (int)(t % kw);
      t /= kw;
      const int ky = (int)(t % kh);
      const int oc = (int)(t / kh);
      s = (((long)oc * ci + i) * kh + ky) * kw + kx;
    } else {
      const int oc = (int)(idx % o);
      const int tap = (int)(idx / o);
      s = (long)oc * kh * kw + tap;
    }
    dst[idx] = from_f32<T>(src[s]);
  }
}

template <typename S, typename D>
__global__ __launch_bounds__(256) void convert_kernel(const S* __restrict__ src,
                                                      D* __restrict__ dst, long n) {
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x)
    dst[idx] = from_f32<D>(to_f32(src[idx]));
}

int grid_for(long total, int cap = 256 * 32) {
  long b = (total + 255) / 256;
  if (b > cap) b = cap;
  if (b < 1) b = 1;
  return (int)b;
}

template <typename T>
int32_t run_pool(const OglePoolArgs& a, hipStream_t s) {
  const T* x = static_cast<const T*>(a.input_dev);
  T* y = static_cast<T*>(a.output_dev);
  const bool whole_image = a.padding == 0 && a.stride == 1 && a.kernel_size == a.in_h &&
                           a.kernel_size == a.in_w && a.pool_type != OGLE_POOL_MAX;
  if (whole_image && a.kernel_size * a.kernel_size >= 16) {
    launch((global_avg_kernel<T>), dim3((a.c + 63) / 64, a.n), dim3(256), 0, s, x, y,
                       a.in_h * a.in_w, a.c);
    return check_launch("global_avg_kernel");
  }
  if constexpr (sizeof(T) == 4) {
    const long total4 = (long)a.n * a.out_h * a.out_w * (a.c / 4);
    const long x_bytes = (long)a.n * a.in_h * a.in_w * a.c * 4, y_bytes = total4 * 16;
    if (a.c % 4 == 0 && (a.kernel_size == 2 || a.kernel_size == 3) && total4 < 0x7fffffffL &&
        x_bytes < 0x7fffffffL && y_bytes < 0x7fffffffL && total4 > 0) {
      const dim3 grid((unsigned)(((total4 + 255) / 256 + 7) / 8 * 8));  // whole XCD rounds
#define OGLE_POOL_SMALL(K)                                                                        \
  launch((pool_small_kernel<K>), grid, dim3(256), 0, s, x, y, a.in_h, a.in_w, a.c,    \
                     a.out_h, a.out_w, a.stride, a.padding, a.pool_type, (unsigned)total4,        \
                     (unsigned)x_bytes, (unsigned)y_bytes, make_pool_div((unsigned)(a.c / 4)),    \
                     make_pool_div((unsigned)a.out_w), make_pool_div((unsigned)a.out_h))
      if (a.kernel_size == 2) OGLE_POOL_SMALL(2);
      else OGLE_POOL_SMALL(3);
#undef OGLE_POOL_SMALL
      return check_launch("pool_small_kernel");
    }
  }
  if (a.c % 4 == 0) {
    const long total = (long)a.n * a.out_h * a.out_w * (a.c / 4);
    launch((pool_kernel<T, 4>), dim3(grid_for(total, 256 * 64)), dim3(256), 0, s, x,
                       y, a.n, a.in_h, a.in_w, a.c, a.out_h, a.out_w, a.kernel_size, a.stride,
                       a.padding, a.pool_type);
  } else {
    const long total = (long)a.n * a.out_h * a.out_w * a.c;
    launch((pool_kernel<T, 1>), dim3(grid_for(total, 256 * 64)), dim3(256), 0, s, x,
                       y, a.n, a.in_h, a.in_w, a.c, a.out_h, a.out_w, a.kernel_size, a.stride,
                       a.padding, a.pool_type);
  }
  return check_launch("pool_kernel");
}

}  // namespace

int32_t launch_pool(const OglePoolArgs& a, hipStream_t s) {
  if (a.dtype == OGLE_F16) return run_pool<__half>(a, s);
  return run_pool<float>(a, s);
}

int32_t launch_concat(const OgleConcatArgs& a, hipStream_t s) {
  const int esz = a.dtype == OGLE_F16 ? 2 : 4;
  const int vec = 16 / esz;
  ConcatPlan p{};
  p.n = a.n_inputs;
  bool vec_ok = (reinterpret_cast<uintptr_t>(a.output_dev) % 16) == 0;
  long off = 0;
  for (int i = 0; i < a.n_inputs; ++i) {
    p.in[i] = a.inputs_dev[i];
    p.run[i] = a.axis_len[i] * a.inner;
    p.start[i] = off;
    off += p.run[i];
    if (p.run[i] % vec != 0 || (reinterpret_cast<uintptr_t>(a.inputs_dev[i]) % 16) != 0)
      vec_ok = false;
  }
  p.out_run = off;
  if (off == 0 || a.outer == 0) return OGLE_OK;
  if (a.outer == 1) {
    // a single outer slice: the output is the inputs back to back, and a caller may
    // have had them produced in place; then there is nothing to move
    bool in_place = true;
    for (int i = 0; i < a.n_inputs; ++i)
      if (p.run[i] > 0 &&
          a.inputs_dev[i] != static_cast<const unsigned char*>(a.output_dev) + p.start[i] * esz)
        in_place = false;
    if (in_place) return OGLE_OK;
  }
  if (vec_ok) {
    for (int i = 0; i < a.n_inputs; ++i) {
      p.run[i] /= vec;
      p.start[i] /= vec;
    }
    p.out_run /= vec;
    p.total = a.outer * p.out_run;
    launch((concat_kernel<uint4>), dim3(grid_for(p.total)), dim3(256), 0, s, p,
                       static_cast<uint4*>(a.output_dev));
  } else if (esz == 4) {
    p.total = a.outer * p.out_run;
    launch((concat_kernel<uint32_t>), dim3(grid_for(p.total)), dim3(256), 0, s, p,
                       static_cast<uint32_t*>(a.output_dev));
  } else {
    p.total = a.outer * p.out_run;
    launch((concat_kernel<uint16_t>), dim3(grid_for(p.total)), dim3(256), 0, s, p,
                       static_cast<uint16_t*>(a.output_dev));
  }
  return check_launch("concat_kernel");
}

int32_t launch_transpose(const OgleTransposeArgs& a, hipStream_t s) {
  TransposePlan p{};
  long stride[4];
  stride[3] = 1;
  for (int d = 2; d >= 0; --d) stride[d] = stride[d + 1] * a.in_shape[d + 1];
  p.total = 1;
  bool identity = true;
  for (int d = 0; d < 4; ++d) {
    p.out_shape[d] = a.in_shape[a.perm[d]];
    p.in_stride[d] = stride[a.perm[d]];
    p.total *= p.out_shape[d];
    // moving a dimension of extent 1 does not change the element order
    if (a.perm[d] != d) identity = false;
  }
  if (p.total == 0) return OGLE_OK;
  if (!identity) {
    // Equivalent to a copy when the non-unit dimensions keep their relative order.
    int last = -1;
    identity = true;
    for (int d = 0; d < 4; ++d) {
      if (p.out_shape[d] == 1) continue;
      if (a.perm[d] < last) identity = false;
      last = a.perm[d];
    }
  }
  const int esz = a.dtype == OGLE_F16 ? 2 : 4;
  if (identity) {
    const hipError_t e = hipMemcpyAsync(a.output_dev, a.input_dev, (size_t)p.total * esz,
                                        hipMemcpyDeviceToDevice, s);
    if (e != hipSuccess) {
      set_error("transpose: copy failed: %s", hipGetErrorString(e));
      return OGLE_ERR_LAUNCH;
    }
    note_launch();
    return OGLE_OK;
  }
  if (esz == 4) {
    launch((transpose_kernel<uint32_t>), dim3(grid_for(p.total)), dim3(256), 0, s, p,
                       static_cast<const uint32_t*>(a.input_dev),
                       static_cast<uint32_t*>(a.output_dev));
  } else {
    launch((transpose_kernel<uint16_t>), dim3(grid_for(p.total)), dim3(256), 0, s, p,
                       static_cast<const uint16_t*>(a.input_dev),
                       static_cast<uint16_t*>(a.output_dev));
  }
  return check_launch("transpose_kernel");
}

int32_t launch_pack_filter(const float* src, void* dst, int layout, int dtype, int o, int i,
                           int kh, int kw, hipStream_t s) {
  const long total = (long)o * i * kh * kw;
  if (total == 0) return OGLE_OK;
  if (dtype == OGLE_F16) {
    launch((pack_filter_kernel<__half>), dim3(grid_for(total)), dim3(256), 0, s, src,
                       static_cast<__half*>(dst), layout, o, i, kh, kw);
  } else {
    launch((pack_filter_kernel<float>), dim3(grid_for(total)), dim3(256), 0, s, src,
                       static_cast<float*>(dst), layout, o, i, kh, kw);
  }
  return check_launch("pack_filter_kernel");
}

int32_t launch_convert(const void* src, int sdt, void* dst, int ddt, int64_t n, hipStream_t s) {
  if (n == 0) return OGLE_OK;
  const dim3 grid(grid_for(n));
  if (sdt == OGLE_F32 && ddt == OGLE_F16) {
    launch((convert_kernel<float, __half>), grid, dim3(256), 0, s,
                       static_cast<const float*>(src), static_cast<__half*>(dst), (long)n);
  } else if (sdt == OGLE_F16 && ddt == OGLE_F32) {
    launch((convert_kernel<__half, float>), grid, dim3(256), 0, s,
                       static_cast<const __half*>(src), static_cast<float*>(dst), (long)n);
  } else if (sdt == OGLE_F32 && ddt == OGLE_F32) {
    launch((convert_kernel<float, float>), grid, dim3(256), 0, s,
                       static_cast<const float*>(src), static_cast<float*>(dst), (long)n);
  } else {
    launch((convert_kernel<__half, __half>), grid, dim3(256), 0, s,
                       static_cast<const __half*>(src), static_cast<__half*>(dst), (long)n);
  }
  return check_launch("convert_kernel");
}

}  // namespace ogle
