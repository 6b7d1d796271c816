/*
 * CPU oracle for the OGLE convolution hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C over dense
 * row-major buffers, the arithmetic that the reference performs in its GLSL
 * fragment shaders and in the host code around them.  It is the checker the
 * HIP kernels are compared with; nothing that ships may link or call it.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference checkout, ogl_runtime/opengl = RT, converter/converter = CV).
 *
 * Pinning status (what each function is checked against, in tests/):
 *   oracle_conv2d        torch.nn.functional.conv2d (CPU, float64), brute-force
 *                        python loops on tiny inputs, all-ones closed form,
 *                        1x1 == matmul, depthwise == scipy correlate2d
 *   oracle_pool2d        F.max_pool2d / F.avg_pool2d(count_include_pad=True),
 *                        window-fully-outside -> 0 special case
 *   oracle_concat        numpy.concatenate, every axis, rank 1..4
 *   oracle_ssd_decode    closed forms (zero prediction -> anchor corners),
 *                        float64 numpy restatement
 *   oracle_box_info      invariants (sum p = 1, id in [1,C-1], strict >),
 *                        float64 numpy softmax
 *   oracle_fold_bn       conv(x; W', b') == BN(conv(x; W, b)) identity
 *   oracle_nchw_to_hwn4c4 / _inverse   round-trip identity + index formula
 *   oracle_topk_nms      brute-force python restatement on small inputs
 *   oracle_add / _relu / _clip   numpy add / maximum / clip
 *   oracle_batchnorm     float64 numpy formula, identity parameters -> x, and
 *                        BN(conv) == conv with oracle_fold_bn's parameters
 *   oracle_gemm          numpy float64 matmul (both transB settings, both bias ranks)
 * No function is "parity unpinned".
 *
 * All arithmetic is IEEE binary32 evaluated in the order the reference uses
 * (ky, kx, then input channel), so results are reproducible bit for bit on
 * any host; build without -ffast-math and without FMA contraction.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_ACT_NONE 0
#define ORACLE_ACT_CLIP 1
#define ORACLE_ACT_RELU 2

/* Shader variants differ only in how the fused activation reads min/max
 * (RT/nn/glsl/conv2d.glsl:82-90, conv2d_pw.glsl:82-90,
 * conv2d_any4.glsl:89-94). */
#define ORACLE_VARIANT_NHWC4 0 /* conv2d.glsl, conv2d_dw.glsl                  */
#define ORACLE_VARIANT_PW 1    /* conv2d_pw.glsl: clamp(x, 0, max)            */
#define ORACLE_VARIANT_ANY4 2  /* *_any4.glsl and conv2d_grp.glsl:115-121:
                                  relu is max(min_value, x)                   */

static inline float oracle_activation(float v, int act, float minv, float maxv,
                                      int variant) {
  if (act == ORACLE_ACT_CLIP) {
    float lo = (variant == ORACLE_VARIANT_PW) ? 0.0f : minv;
    /* GLSL clamp(x, lo, hi) == min(max(x, lo), hi) */
    v = v < lo ? lo : v;
    v = v > maxv ? maxv : v;
  } else if (act == ORACLE_ACT_RELU) {
    float lo = (variant == ORACLE_VARIANT_ANY4) ? minv : 0.0f;
    v = v < lo ? lo : v;
  }
  return v;
}

/* Output spatial size.  RT/nn/kernels/conv2d.cc:191-193 (conv),
 * RT/nn/kernels/pool.cc:94-96 (pool, dilation 1). */
int oracle_out_size(int in, int k, int stride, int pad, int dilation) {
  int keff = k * dilation - dilation + 1;
  return (in - keff + 2 * pad) / stride + 1;
}

/*
 * Direct convolution, NHWC input, OIHW filter (O, C/groups, k, k), NHWC output.
 * Restates Conv2DCPU (RT/nn/kernels/conv2d_test.cc:18-75), extended over the
 * batch, with the bias-first accumulation and the fused activation of the
 * shaders (RT/nn/glsl/conv2d.glsl:42-90, conv2d_dw.glsl:51-95,
 * conv2d_pw.glsl:50-90).  Accumulation order: bias, then ky, kx, c ascending.
 * Out-of-image taps are skipped (zero padding).
 */
void oracle_conv2d(const float* x, const float* w, const float* bias, float* y,
                   int n, int h, int wd, int c, int o, int k, int stride,
                   int pad, int dilation, int groups, int act, float minv,
                   float maxv, int variant) {
  const int oh = oracle_out_size(h, k, stride, pad, dilation);
  const int ow = oracle_out_size(wd, k, stride, pad, dilation);
  const int cpg = c / groups;
  const int opg = o / groups;
  const long rows = (long)n * oh;
#pragma omp parallel for schedule(static)
  for (long row = 0; row < rows; ++row) {
    const int b = (int)(row / oh);
    const int oy = (int)(row % oh);
    for (int ox = 0; ox < ow; ++ox) {
      float* yp = y + (((long)b * oh + oy) * ow + ox) * o;
      for (int oc = 0; oc < o; ++oc) {
        const int g = oc / opg;
        const float* wf = w + (long)oc * cpg * k * k;
        float sum = bias ? bias[oc] : 0.0f;
        for (int r = 0; r < k; ++r) {
          const int iy = oy * stride - pad + r * dilation;
          if (iy < 0 || iy >= h) continue;
          for (int s = 0; s < k; ++s) {
            const int ix = ox * stride - pad + s * dilation;
            if (ix < 0 || ix >= wd) continue;
            const float* xp = x + (((long)b * h + iy) * wd + ix) * c + g * cpg;
            const int tap = r * k + s;
            for (int ci = 0; ci < cpg; ++ci) {
              sum += xp[ci] * wf[ci * k * k + tap];
            }
          }
        }
        yp[oc] = oracle_activation(sum, act, minv, maxv, variant);
      }
    }
  }
}

/*
 * Same contraction with |x| and |w| (and |bias|): the magnitude each output's
 * rounding error is proportional to.  Used by the tests to express the fp32
 * tolerance relative to the accumulated magnitude.  No reference counterpart.
 */
void oracle_conv2d_abs(const float* x, const float* w, const float* bias,
                       float* y, int n, int h, int wd, int c, int o, int k,
                       int stride, int pad, int dilation, int groups) {
  const int oh = oracle_out_size(h, k, stride, pad, dilation);
  const int ow = oracle_out_size(wd, k, stride, pad, dilation);
  const int cpg = c / groups;
  const int opg = o / groups;
  const long rows = (long)n * oh;
#pragma omp parallel for schedule(static)
  for (long row = 0; row < rows; ++row) {
    const int b = (int)(row / oh);
    const int oy = (int)(row % oh);
    for (int ox = 0; ox < ow; ++ox) {
      float* yp = y + (((long)b * oh + oy) * ow + ox) * o;
      for (int oc = 0; oc < o; ++oc) {
        const int g = oc / opg;
        const float* wf = w + (long)oc * cpg * k * k;
        float sum = bias ? fabsf(bias[oc]) : 0.0f;
        for (int r = 0; r < k; ++r) {
          const int iy = oy * stride - pad + r * dilation;
          if (iy < 0 || iy >= h) continue;
          for (int s = 0; s < k; ++s) {
            const int ix = ox * stride - pad + s * dilation;
            if (ix < 0 || ix >= wd) continue;
            const float* xp = x + (((long)b * h + iy) * wd + ix) * c + g * cpg;
            const int tap = r * k + s;
            for (int ci = 0; ci < cpg; ++ci) {
              sum += fabsf(xp[ci]) * fabsf(wf[ci * k * k + tap]);
            }
          }
        }
        yp[oc] = sum;
      }
    }
  }
}

/*
 * Pooling over NHWC.  Restates RT/nn/glsl/pool.glsl:19-66 with the output
 * shape of RT/nn/kernels/pool.cc:84-96.  pool_type 0 = max, 1 = average,
 * 2 = global average (RT/nn/kernels/pool.h:10-14); for type 2 the caller
 * passes k = H, stride 1, pad 0 as PoolKernel::InferOutputShape sets them.
 * Max: the first in-image tap initialises, later ones take max; a window with
 * no in-image tap yields 0.  Average: sum of in-image taps divided by k*k
 * always.  Tap order: kx outer, ky inner (pool.glsl:31-32).
 */
void oracle_pool2d(const float* x, float* y, int n, int h, int wd, int c, int k,
                   int stride, int pad, int pool_type) {
  const int oh = oracle_out_size(h, k, stride, pad, 1);
  const int ow = oracle_out_size(wd, k, stride, pad, 1);
  const long rows = (long)n * oh;
#pragma omp parallel for schedule(static)
  for (long row = 0; row < rows; ++row) {
    const int b = (int)(row / oh);
    const int oy = (int)(row % oh);
    for (int ox = 0; ox < ow; ++ox) {
      float* yp = y + (((long)b * oh + oy) * ow + ox) * c;
      for (int ch = 0; ch < c; ++ch) {
        float v = 0.0f;
        int first = 1;
        for (int i = 0; i < k; ++i) {
          const int ix = ox * stride + i - pad;
          if (ix < 0 || ix >= wd) continue;
          for (int j = 0; j < k; ++j) {
            const int iy = oy * stride + j - pad;
            if (iy < 0 || iy >= h) continue;
            const float item = x[(((long)b * h + iy) * wd + ix) * c + ch];
            if (pool_type == 0) {
              if (first) {
                v = item;
                first = 0;
              } else {
                v = v > item ? v : item;
              }
            } else {
              v += item;
            }
          }
        }
        if (pool_type != 0) v = v / (float)(k * k);
        yp[ch] = v;
      }
    }
  }
}

/*
 * N-input concatenation along `axis` of row-major tensors of equal rank
 * (rank <= 8).  Restates ConcatCPU (RT/nn/kernels/concat_test.cc:9-34)
 * generalised to n inputs as ConcatKernel::Compute applies it
 * (RT/nn/kernels/concat.cc:56-97): each input occupies
 * [axis_offset, axis_offset + len) of the output's axis.  The element values
 * are copied, so the result is exact.  shapes is n_inputs x rank.
 * Returns 0, or -1 if a non-axis dimension differs
 * (RT/nn/kernels/concat.cc:116-121).
 */
int oracle_concat(const float* const* inputs, const int* shapes, int n_inputs,
                  int rank, int axis, float* out) {
  if (axis < 0) axis += rank; /* concat.cc:105-107 */
  if (axis < 0 || axis >= rank || rank > 8) return -1;
  long outer = 1, inner = 1;
  for (int d = 0; d < axis; ++d) outer *= shapes[d];
  for (int d = axis + 1; d < rank; ++d) inner *= shapes[d];
  long total_axis = 0;
  for (int i = 0; i < n_inputs; ++i) {
    for (int d = 0; d < rank; ++d) {
      if (d != axis && shapes[i * rank + d] != shapes[d]) return -1;
    }
    total_axis += shapes[i * rank + axis];
  }
  long axis_offset = 0;
  for (int i = 0; i < n_inputs; ++i) {
    const long len = shapes[i * rank + axis];
    for (long ob = 0; ob < outer; ++ob) {
      memcpy(out + (ob * total_axis + axis_offset) * inner,
             inputs[i] + ob * len * inner, sizeof(float) * len * inner);
    }
    axis_offset += len;
  }
  return 0;
}

/*
 * SSD box decode: center-size anchors and predictions to corner boxes.
 * Restates host_functor::SSDBBoxDecoder (RT/core/cpu_functor.cc:129-154),
 * which is the reference's own CPU twin of RT/nn/glsl/decoder.glsl:13-28,
 * extended over the batch with the anchors shared by every image.  The host
 * functor multiplies by the double literal 0.5 and narrows on assignment;
 * that is kept.  pred (batch, priors, 4), anchors (priors, 4) as
 * (cx, cy, w, h); out (batch, priors, 4) as (xmin, ymin, xmax, ymax).
 */
void oracle_ssd_decode(const float* pred, const float* anchors, float* out,
                       int batch, int priors, const float* variances) {
  for (int b = 0; b < batch; ++b) {
    const float* p = pred + (long)b * priors * 4;
    float* d = out + (long)b * priors * 4;
    for (int i = 0; i < priors; ++i) {
      const float* a = anchors + (long)i * 4;
      float ycenter = p[i * 4 + 1] * variances[1] * a[3] + a[1];
      float xcenter = p[i * 4 + 0] * variances[0] * a[2] + a[0];
      float hh = expf(p[i * 4 + 3] * variances[3]) * a[3];
      float ww = expf(p[i * 4 + 2] * variances[2]) * a[2];
      float ymin = (float)(ycenter - hh * 0.5);
      float xmin = (float)(xcenter - ww * 0.5);
      float ymax = (float)(ycenter + hh * 0.5);
      float xmax = (float)(xcenter + ww * 0.5);
      d[i * 4 + 0] = xmin;
      d[i * 4 + 1] = ymin;
      d[i * 4 + 2] = xmax;
      d[i * 4 + 3] = ymax;
    }
  }
}

/*
 * Per-prior class score and threshold: restates Detector::GenerateBoxInfo
 * (RT/examples/ssd/detector.cc:184-225) for every image of the batch.
 * sum = expf(l0); for j = 1..C-1: e = expf(lj), sum += e, strict-greater max
 * starting from 0 (so class 0, background, is never chosen unless every e is
 * 0).  p = e_max / sum; kept iff p > threshold (strict).
 * Boxes (corner form, normalised) are scaled by the image size in fp32
 * (detector.cc:201-204) and, as cv::Rect is integer, x, y, width, height are
 * truncated toward zero on assignment (detector.cc:211-214).
 *
 * Outputs per image b, compacted in ascending prior order:
 *   kept_count[b]; kept_prior[b*priors + r]; kept_class[...]; kept_score[...];
 *   kept_box[(b*priors + r)*4 + {0..3}] = scaled xmin, ymin, xmax, ymax (fp32);
 *   kept_rect[(b*priors + r)*4 + {0..3}] = int x, y, width, height.
 * Any output pointer except kept_count may be NULL.
 */
void oracle_box_info(const float* logits, const float* boxes, int batch,
                     int priors, int classes, float threshold, float image_w,
                     float image_h, int32_t* kept_count, int32_t* kept_prior,
                     int32_t* kept_class, float* kept_score, float* kept_box,
                     int32_t* kept_rect) {
  for (int b = 0; b < batch; ++b) {
    int r = 0;
    for (int i = 0; i < priors; ++i) {
      const float* l = logits + ((long)b * priors + i) * classes;
      float total_sum = expf(l[0]);
      int max_id = 0;
      float max_prob = 0.0f;
      for (int j = 1; j < classes; ++j) {
        float e = expf(l[j]);
        total_sum += e;
        if (max_prob < e) {
          max_prob = e;
          max_id = j;
        }
      }
      const float* bx = boxes + ((long)b * priors + i) * 4;
      float xmin = bx[0] * image_w;
      float ymin = bx[1] * image_h;
      float xmax = bx[2] * image_w;
      float ymax = bx[3] * image_h;
      max_prob /= total_sum;
      if (max_prob > threshold) {
        const long slot = (long)b * priors + r;
        if (kept_prior) kept_prior[slot] = i;
        if (kept_class) kept_class[slot] = max_id;
        if (kept_score) kept_score[slot] = max_prob;
        if (kept_box) {
          kept_box[slot * 4 + 0] = xmin;
          kept_box[slot * 4 + 1] = ymin;
          kept_box[slot * 4 + 2] = xmax;
          kept_box[slot * 4 + 3] = ymax;
        }
        if (kept_rect) {
          kept_rect[slot * 4 + 0] = (int32_t)xmin;
          kept_rect[slot * 4 + 1] = (int32_t)ymin;
          kept_rect[slot * 4 + 2] = (int32_t)(xmax - xmin);
          kept_rect[slot * 4 + 3] = (int32_t)(ymax - ymin);
        }
        ++r;
      }
    }
    kept_count[b] = r;
  }
}

/* expf exactly as the oracle evaluates it, exposed so a GPU test can compare
 * the device exponential with the host libm on the same inputs. */
void oracle_expf_array(const float* x, float* y, long n) {
  for (long i = 0; i < n; ++i) y[i] = expf(x[i]);
}

/*
 * Batch-norm folding into a convolution: restates
 * MergeBatchNormToConvolution (CV/optimizers/remapper.cc:142-149).
 * scale = gamma / sqrt(var + eps) in fp32 (std::sqrt on float);
 * w[o, :] *= scale; b[o] = b[o] * scale + (-scale * mean + beta).
 * If the conv had no bias the caller passes a zero bias
 * (remapper.cc:124-134).  w is (O, chw) row-major, modified in place.
 */
void oracle_fold_bn(float* w, float* bias, const float* gamma,
                    const float* beta, const float* mean, const float* var,
                    float eps, int o, int chw) {
  for (int i = 0; i < o; ++i) {
    float scale = gamma[i] / sqrtf(var[i] + eps);
    float shift = -scale * mean[i] + beta[i];
    for (int j = 0; j < chw; ++j) w[(long)i * chw + j] *= scale;
    bias[i] = bias[i] * scale + shift;
  }
}

/*
 * The reference's filter texture layout, as a flat float array:
 * OIHW (n_out, n_in, h, w) -> HWN4C4 with texel (x = i, y = (ky*kw+kx)*O4 +
 * o/4), lane o%4; rows are IN4*4 texels wide (RT/core/tensor_format.cc:289-295,
 * 338-343; host form RT/core/cpu_functor.cc:87-116).  dst holds
 * h*w*O4 * I4*4 * 4 floats, zero filled where o or i is padding.
 */
void oracle_nchw_to_hwn4c4(const float* src, float* dst, int n_out, int n_in,
                           int kh, int kw) {
  const int o4 = (n_out + 3) / 4;
  const int i4 = (n_in + 3) / 4;
  const long width = (long)i4 * 4;
  memset(dst, 0, sizeof(float) * kh * kw * o4 * width * 4);
  for (int o = 0; o < n_out; ++o)
    for (int i = 0; i < n_in; ++i)
      for (int ky = 0; ky < kh; ++ky)
        for (int kx = 0; kx < kw; ++kx) {
          long ytex = (long)(ky * kw + kx) * o4 + o / 4;
          long di = (ytex * width + i) * 4 + o % 4;
          dst[di] = src[(((long)o * n_in + i) * kh + ky) * kw + kx];
        }
}

void oracle_hwn4c4_to_nchw(const float* src, float* dst, int n_out, int n_in,
                           int kh, int kw) {
  const int o4 = (n_out + 3) / 4;
  const int i4 = (n_in + 3) / 4;
  const long width = (long)i4 * 4;
  for (int o = 0; o < n_out; ++o)
    for (int i = 0; i < n_in; ++i)
      for (int ky = 0; ky < kh; ++ky)
        for (int kx = 0; kx < kw; ++kx) {
          long ytex = (long)(ky * kw + kx) * o4 + o / 4;
          long si = (ytex * width + i) * 4 + o % 4;
          dst[(((long)o * n_in + i) * kh + ky) * kw + kx] = src[si];
        }
}

/*
 * IoU on integer rectangles (x, y, width, height), restating iou()
 * (RT/examples/ssd/common.cc:57-77).
 */
static float oracle_iou(const int32_t* r0, const int32_t* r1) {
  float xmin0 = (float)r0[0], ymin0 = (float)r0[1];
  float xmax0 = (float)(r0[0] + r0[2]), ymax0 = (float)(r0[1] + r0[3]);
  float xmin1 = (float)r1[0], ymin1 = (float)r1[1];
  float xmax1 = (float)(r1[0] + r1[2]), ymax1 = (float)(r1[1] + r1[3]);
  float w = fmaxf(0.0f, fminf(xmax0, xmax1) - fmaxf(xmin0, xmin1));
  float h = fmaxf(0.0f, fminf(ymax0, ymax1) - fmaxf(ymin0, ymin1));
  float i = w * h;
  float u = (xmax0 - xmin0) * (ymax0 - ymin0) +
            (xmax1 - xmin1) * (ymax1 - ymin1) - i;
  if (u <= 0.0f) return 0.0f;
  return i / u;
}

/*
 * Top-k then NMS for one image: restates Detector::GetTopK
 * (RT/examples/ssd/detector.cc:114-125) and Detector::NMS
 * (detector.cc:127-148).  The reference sorts with std::sort (unstable) by
 * score descending; here ties are broken by ascending input position so the
 * result is defined.  Suppression: box j is dropped if ANY earlier box i
 * (i < j in sorted order) overlaps it by more than nms_threshold, even when i
 * was itself dropped.  order_out receives the input positions of the
 * survivors in sorted order; returns their number.
 */
int oracle_topk_nms(const float* scores, const int32_t* rects, int count,
                    int top_k, float nms_threshold, int32_t* order_out) {
  int32_t* idx = (int32_t*)malloc(sizeof(int32_t) * (count > 0 ? count : 1));
  for (int i = 0; i < count; ++i) idx[i] = i;
  /* insertion sort: stable, descending score */
  for (int i = 1; i < count; ++i) {
    int32_t v = idx[i];
    int j = i - 1;
    while (j >= 0 && scores[idx[j]] < scores[v]) {
      idx[j + 1] = idx[j];
      --j;
    }
    idx[j + 1] = v;
  }
  int m = count < top_k ? count : top_k;
  char* dropped = (char*)calloc(m > 0 ? m : 1, 1);
  for (int i = 0; i < m - 1; ++i)
    for (int j = i + 1; j < m; ++j)
      if (oracle_iou(rects + 4 * (long)idx[i], rects + 4 * (long)idx[j]) >
          nms_threshold)
        dropped[j] = 1;
  int out = 0;
  for (int i = 0; i < m; ++i)
    if (!dropped[i]) order_out[out++] = idx[i];
  free(idx);
  free(dropped);
  return out;
}

/* ---- elementwise ops and Gemm of classification graphs ---------------------- */

/* RT/nn/glsl/binary.glsl:8: texel-wise sum of two tensors of one shape. */
void oracle_add(const float* a, const float* b, float* y, long n) {
  for (long i = 0; i < n; ++i) y[i] = a[i] + b[i];
}

/* RT/nn/glsl/relu.glsl:8-10. */
void oracle_relu(const float* x, float* y, long n) {
  for (long i = 0; i < n; ++i) y[i] = x[i] > 0.0f ? x[i] : 0.0f;
}

/* RT/nn/glsl/clip.glsl:7-12: max with min_value first, then min with max_value. */
void oracle_clip(const float* x, float* y, long n, float minv, float maxv) {
  for (long i = 0; i < n; ++i) {
    float v = x[i];
    v = minv > v ? minv : v;
    v = maxv < v ? maxv : v;
    y[i] = v;
  }
}

/* RT/nn/glsl/batchnorm.glsl:33: (x - mean) / sqrt(var + eps) * gamma + beta with the
 * parameters indexed by the last (channel) dimension, evaluated left to right. */
void oracle_batchnorm(const float* x, const float* gamma, const float* beta, const float* mean,
                      const float* var, float* y, long outer, int channels, float eps) {
  for (long i = 0; i < outer; ++i)
    for (int c = 0; c < channels; ++c) {
      const float d = x[i * channels + c] - mean[c];
      const float q = d / sqrtf(var[c] + eps);
      y[i * channels + c] = q * gamma[c] + beta[c];
    }
}

/* RT/nn/glsl/gemm.glsl:33-95 with GemmCPU's reading of C (RT/nn/kernels/gemm_test.cc:9-40):
 * y[i][j] = sum_m alpha * a[i][m] * b(m, j), terms added for m ascending, then
 * + beta * c.  b is (N, K) when trans_b, (K, N) otherwise.  c is NULL, a row of N
 * values broadcast over the rows (c_rank 1), or (M, N) (c_rank 2). */
void oracle_gemm(const float* a, const float* b, const float* c, float* y, int m_rows, int n_cols,
                 int k, int trans_b, int c_rank, float alpha, float beta) {
  for (int i = 0; i < m_rows; ++i)
    for (int j = 0; j < n_cols; ++j) {
      float acc = 0.0f;
      for (int m = 0; m < k; ++m) {
        const float bv = trans_b ? b[(long)j * k + m] : b[(long)m * n_cols + j];
        acc += alpha * a[(long)i * k + m] * bv;
      }
      if (c != NULL) acc += beta * (c_rank == 2 ? c[(long)i * n_cols + j] : c[j]);
      y[(long)i * n_cols + j] = acc;
    }
}

/* Number of threads the OpenMP loops above will use (for bench.py's report). */
#ifdef _OPENMP
#include <omp.h>
int oracle_num_threads(void) { return omp_get_max_threads(); }
#else
int oracle_num_threads(void) { return 1; }
#endif
