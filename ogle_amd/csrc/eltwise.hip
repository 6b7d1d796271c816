// Elementwise ops of classification graphs and the Gemm at their end:
// Add (binary.glsl:8), Relu (relu.glsl:8-10), Clip (clip.glsl:7-12),
// BatchNormalization (batchnorm.glsl:33) and Gemm (gemm.glsl:33-95).  All are
// bandwidth bound: a thread moves 16 bytes per access, a grid-stride loop covers the
// tensor, and the arithmetic keeps the shaders' operation order (no FMA contraction,
// IEEE division and square root) so results match the CPU restatement bit for bit
// in fp32 (Gemm: to the contraction tolerance).
#include "common.h"

namespace ogle {

namespace {

constexpr int kVec = 4;  // elements per thread and access (16 bytes of fp32, 8 of fp16)

template <typename T>
struct Vec4;
template <>
struct Vec4<float> {
  typedef float4 type;
  __device__ static __forceinline__ void load(const float* p, float v[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ static __forceinline__ void store(float* p, const float v[4]) {
    store_result16(p, make_float4(v[0], v[1], v[2], v[3]));
  }
};
template <>
struct Vec4<__half> {
  __device__ static __forceinline__ void load(const __half* p, float v[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    const __half2 lo = *reinterpret_cast<const __half2*>(&t.x);
    const __half2 hi = *reinterpret_cast<const __half2*>(&t.y);
    v[0] = __low2float(lo); v[1] = __high2float(lo); v[2] = __low2float(hi); v[3] = __high2float(hi);
  }
  __device__ static __forceinline__ void store(__half* p, const float v[4]) {
    const __half2 lo = __floats2half2_rn(v[0], v[1]), hi = __floats2half2_rn(v[2], v[3]);
    uint2 t;
    t.x = *reinterpret_cast<const unsigned*>(&lo);
    t.y = *reinterpret_cast<const unsigned*>(&hi);
    store_result8(p, t);
  }
};

struct UnaryOp {
  int op;
  float lo, hi;
  __device__ __forceinline__ float operator()(float v) const {
    if (op == OGLE_UNARY_RELU) return v > 0.f ? v : 0.f;
    v = lo > v ? lo : v;   // clip.glsl: max with min_value first,
    return hi < v ? hi : v;  // then min with max_value
  }
};

template <typename T>
__global__ __launch_bounds__(256) void unary_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                    long n, UnaryOp f) {
  const long vecs = n / kVec;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < vecs;
       i += (long)gridDim.x * blockDim.x) {
    float v[4];
    Vec4<T>::load(x + i * kVec, v);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = f(v[j]);
    Vec4<T>::store(y + i * kVec, v);
  }
  // the last n % 4 elements
  const long tail = vecs * kVec + (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (tail < n) y[tail] = from_f32<T>(f(to_f32(x[tail])));
}

template <typename T>
__global__ __launch_bounds__(256) void add_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                  T* __restrict__ y, long n) {
  const long vecs = n / kVec;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < vecs;
       i += (long)gridDim.x * blockDim.x) {
    float u[4], v[4];
    Vec4<T>::load(a + i * kVec, u);
    Vec4<T>::load(b + i * kVec, v);
#pragma unroll
    for (int j = 0; j < 4; ++j) u[j] += v[j];
    Vec4<T>::store(y + i * kVec, u);
  }
  const long tail = vecs * kVec + (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (tail < n) y[tail] = from_f32<T>(to_f32(a[tail]) + to_f32(b[tail]));
}

#pragma clang fp contract(off)
__device__ __forceinline__ float bn_one(float x, float gamma, float beta, float mean, float var,
                                        float eps) {
  // (x - mean) / sqrt(var + eps) * gamma + beta, left to right, every step rounded
  // (sqrtf and / are the correctly rounded forms; the __f*_rn intrinsics are not all)
  const float d = x - mean;
  const float q = d / sqrtf(var + eps);
  return q * gamma + beta;
}

// Channels are the last dimension.  VEC = 4: C % 4 == 0, a thread owns four channels.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void batchnorm_kernel(
    const T* __restrict__ x, const float* __restrict__ gamma, const float* __restrict__ beta,
    const float* __restrict__ mean, const float* __restrict__ var, T* __restrict__ y, long total,
    int channels, float eps) {
  const long items = total / VEC;
  const int cvec = channels / VEC;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < items;
       i += (long)gridDim.x * blockDim.x) {
    const int c0 = (int)(i % cvec) * VEC;
    if constexpr (VEC == 4) {
      float v[4];
      Vec4<T>::load(x + i * 4, v);
      const float4 g = *reinterpret_cast<const float4*>(gamma + c0);
      const float4 bt = *reinterpret_cast<const float4*>(beta + c0);
      const float4 mu = *reinterpret_cast<const float4*>(mean + c0);
      const float4 vr = *reinterpret_cast<const float4*>(var + c0);
      v[0] = bn_one(v[0], g.x, bt.x, mu.x, vr.x, eps);
      v[1] = bn_one(v[1], g.y, bt.y, mu.y, vr.y, eps);
      v[2] = bn_one(v[2], g.z, bt.z, mu.z, vr.z, eps);
      v[3] = bn_one(v[3], g.w, bt.w, mu.w, vr.w, eps);
      Vec4<T>::store(y + i * 4, v);
    } else {
      y[i] = from_f32<T>(bn_one(to_f32(x[i]), gamma[c0], beta[c0], mean[c0], var[c0], eps));
    }
  }
}

// General Gemm: a 16 x 64 tile of Y per workgroup, K walked in chunks of 32 through
// LDS.  Takes what the MFMA kernel does not (B not transposed, alpha or beta other
// than 1, a full (M, N) addend, K not a multiple of 4).
constexpr int kGemmBM = 16, kGemmBN = 64, kGemmBK = 32;

__global__ __launch_bounds__(256) void gemm_general_kernel(
    const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ c,
    float* __restrict__ y, int m, int n, int k, int trans_b, int c_rank, float alpha, float beta) {
  __shared__ float sa[kGemmBM][kGemmBK + 1];
  __shared__ float sb[kGemmBK][kGemmBN + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;  // thread: row ty, columns tx, tx+16, tx+32, tx+48
  const int m0 = blockIdx.y * kGemmBM, n0 = blockIdx.x * kGemmBN;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k; k0 += kGemmBK) {
    for (int i = tid; i < kGemmBM * kGemmBK; i += 256) {
      const int r = i / kGemmBK, kk = i % kGemmBK;
      sa[r][kk] = (m0 + r < m && k0 + kk < k) ? a[(long)(m0 + r) * k + k0 + kk] : 0.f;
    }
    for (int i = tid; i < kGemmBK * kGemmBN; i += 256) {
      int kk, col;
      if (trans_b) {  // B is (N, K): consecutive threads along K
        col = i / kGemmBK;
        kk = i % kGemmBK;
      } else {        // B is (K, N): consecutive threads along N
        kk = i / kGemmBN;
        col = i % kGemmBN;
      }
      float v = 0.f;
      if (n0 + col < n && k0 + kk < k)
        v = trans_b ? b[(long)(n0 + col) * k + k0 + kk] : b[(long)(k0 + kk) * n + n0 + col];
      sb[kk][col] = v;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < kGemmBK; ++kk) {
      const float av = sa[ty][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += av * sb[kk][tx + 16 * j];
    }
    __syncthreads();
  }
  const int row = m0 + ty;
  if (row >= m) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = n0 + tx + 16 * j;
    if (col >= n) continue;
    float v = alpha * acc[j];
    if (c != nullptr) v += beta * (c_rank == 2 ? c[(long)row * n + col] : c[col]);
    y[(long)row * n + col] = v;
  }
}

int grid_for(long items) {
  long b = (items + 255) / 256;
  if (b > 256 * 32) b = 256 * 32;
  if (b < 1) b = 1;
  return (int)b;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

int32_t launch_unary(const OgleUnaryArgs& a, hipStream_t s) {
  if (a.count == 0) return OGLE_OK;
  const UnaryOp f{a.op, a.min_value, a.max_value};
  const dim3 grid(grid_for(a.count / kVec + 1));
  if (a.dtype == OGLE_F16) {
    launch((unary_kernel<__half>), grid, dim3(256), 0, s,
                       static_cast<const __half*>(a.input_dev), static_cast<__half*>(a.output_dev),
                       (long)a.count, f);
  } else {
    launch((unary_kernel<float>), grid, dim3(256), 0, s,
                       static_cast<const float*>(a.input_dev), static_cast<float*>(a.output_dev),
                       (long)a.count, f);
  }
  return check_launch("unary_kernel");
}

int32_t launch_binary(const OgleBinaryArgs& a, hipStream_t s) {
  if (a.count == 0) return OGLE_OK;
  const dim3 grid(grid_for(a.count / kVec + 1));
  if (a.dtype == OGLE_F16) {
    launch((add_kernel<__half>), grid, dim3(256), 0, s,
                       static_cast<const __half*>(a.a_dev), static_cast<const __half*>(a.b_dev),
                       static_cast<__half*>(a.output_dev), (long)a.count);
  } else {
    launch((add_kernel<float>), grid, dim3(256), 0, s,
                       static_cast<const float*>(a.a_dev), static_cast<const float*>(a.b_dev),
                       static_cast<float*>(a.output_dev), (long)a.count);
  }
  return check_launch("add_kernel");
}

int32_t launch_batchnorm(const OgleBatchNormArgs& a, hipStream_t s) {
  const long total = (long)a.outer * a.channels;
  if (total == 0) return OGLE_OK;
  const bool vec = a.channels % 4 == 0 && aligned16(a.gamma_dev) && aligned16(a.beta_dev) &&
                   aligned16(a.mean_dev) && aligned16(a.var_dev);
  const dim3 grid(grid_for(vec ? total / 4 : total));
#define OGLE_BN_LAUNCH(T, VEC)                                                                   \
  launch((batchnorm_kernel<T, VEC>), grid, dim3(256), 0, s,                          \
                     static_cast<const T*>(a.input_dev), a.gamma_dev, a.beta_dev, a.mean_dev,    \
                     a.var_dev, static_cast<T*>(a.output_dev), total, a.channels, a.epsilon)
  if (a.dtype == OGLE_F16) {
    if (vec) OGLE_BN_LAUNCH(__half, 4);
    else OGLE_BN_LAUNCH(__half, 1);
  } else {
    if (vec) OGLE_BN_LAUNCH(float, 4);
    else OGLE_BN_LAUNCH(float, 1);
  }
#undef OGLE_BN_LAUNCH
  return check_launch("batchnorm_kernel");
}

// The Linear-layer form (B transposed, alpha = 1, addend a row with beta = 1 or
// absent, K % 4 == 0) is a pointwise convolution over M "pixels": it goes to the MFMA
// implicit-GEMM kernel, whose split-K plans cover the small M of a classifier head.
static bool gemm_is_pointwise(const OgleGemmArgs& a) {
  return a.trans_b != 0 && a.alpha == 1.f && a.k % 4 == 0 &&
         (a.c_dev == nullptr || (a.c_rank == 1 && a.beta == 1.f));
}

static OgleConvArgs gemm_as_conv(const OgleGemmArgs& a) {
  OgleConvArgs c{};
  c.input_dev = a.a_dev;
  c.filter_dev = a.b_dev;
  c.bias_dev = a.c_dev;
  c.output_dev = a.y_dev;
  c.n = a.m; c.in_h = 1; c.in_w = 1; c.in_c = a.k;
  c.out_h = 1; c.out_w = 1; c.out_c = a.n;
  c.kernel_size = 1; c.stride = 1; c.padding = 0; c.dilation = 1; c.group = 1;
  c.act = OGLE_ACT_NONE;
  c.act_variant = OGLE_VARIANT_PW;
  c.dtype = OGLE_F32;
  c.workspace_dev = a.workspace_dev;
  c.workspace_bytes = a.workspace_bytes;
  return c;
}

size_t gemm_workspace_bytes(const OgleGemmArgs& a) {
  if (!gemm_is_pointwise(a)) return 0;
  return conv_igemm_workspace_bytes(gemm_as_conv(a));
}

int32_t launch_gemm(const OgleGemmArgs& a, hipStream_t s) {
  if (a.m == 0 || a.n == 0) return OGLE_OK;
  if (gemm_is_pointwise(a)) {
    const int32_t st = launch_conv_igemm(gemm_as_conv(a), s);
    if (st != OGLE_ERR_UNSUPPORTED) return st;
  }
  const dim3 grid((a.n + kGemmBN - 1) / kGemmBN, (a.m + kGemmBM - 1) / kGemmBM);
  launch(gemm_general_kernel, grid, dim3(256), 0, s, a.a_dev, a.b_dev, a.c_dev, a.y_dev,
                     a.m, a.n, a.k, a.trans_b, a.c_rank, a.alpha, a.beta);
  return check_launch("gemm_general_kernel");
}

}  // namespace ogle
