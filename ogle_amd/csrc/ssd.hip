// SSD box decoder and score filter.
//
// ssd_decode_kernel restates decoder.glsl:13-28 (center-size -> corners with
// variances).  ssd_detect_kernel fuses it with the per-prior work of
// Detector::GenerateBoxInfo (examples/ssd/detector.cc:184-225): sequential fp32
// softmax denominator over classes 0..C-1, strict-greater maximum over classes
// 1..C-1, p = e_max / sum, keep iff p > threshold, scale to pixels, truncate to
// an integer rectangle; kept priors are written compacted in ascending prior
// order (the order the host loop produces them in).
//
// Every floating-point operation here is a separate IEEE binary32 operation in
// the host code's order: contraction into FMA is disabled for this file, and
// exp is evaluated in binary64 and rounded once to binary32, i.e. a correctly
// rounded expf, which is what the host's libm returns in all but a vanishing
// fraction of inputs.  That keeps kept indices and class ids equal to the host
// result bit for bit.
#pragma clang fp contract(off)
#include "common.h"

namespace ogle {
namespace {

__device__ __forceinline__ float exp_cr(float v) { return (float)exp((double)v); }

__device__ __forceinline__ float4 decode_one(const float4 p, const float4 a, const float v0,
                                             const float v1, const float v2, const float v3) {
  const float ycenter = p.y * v1 * a.w + a.y;
  const float xcenter = p.x * v0 * a.z + a.x;
  const float hh = exp_cr(p.w * v3) * a.w;
  const float ww = exp_cr(p.z * v2) * a.z;
  // The host narrows (double)center -/+ (double)size*0.5 to float.
  float4 o;
  o.y = (float)((double)ycenter - (double)hh * 0.5);
  o.x = (float)((double)xcenter - (double)ww * 0.5);
  o.w = (float)((double)ycenter + (double)hh * 0.5);
  o.z = (float)((double)xcenter + (double)ww * 0.5);
  return o;
}

__global__ __launch_bounds__(256) void ssd_decode_kernel(const float4* __restrict__ pred,
                                                         const float4* __restrict__ anchors,
                                                         float4* __restrict__ out, int batch,
                                                         int priors, long anchor_stride_vec,
                                                         float v0, float v1, float v2, float v3) {
  const long total = (long)batch * priors;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int b = (int)(idx / priors);
    const int i = (int)(idx - (long)b * priors);
    out[idx] = decode_one(pred[idx], anchors[b * anchor_stride_vec + i], v0, v1, v2, v3);
  }
}

__global__ __launch_bounds__(256) void expf_kernel(const float* __restrict__ x,
                                                   float* __restrict__ y, long n) {
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x)
    y[idx] = exp_cr(x[idx]);
}

struct DetectParams {
  const float* logits;
  const float4* pred;
  const float4* anchors;
  float4* boxes;
  int batch, priors, classes;
  long anchor_stride_vec;
  float v0, v1, v2, v3;
  float threshold, image_w, image_h;
  int32_t* kept_count;
  int32_t* kept_prior;
  int32_t* kept_class;
  float* kept_score;
  float4* kept_box;
  int4* kept_rect;
};

// One workgroup per image walks the priors in slabs of 256.  A slab's logits
// (256 x classes floats, contiguous) are staged into LDS with coalesced loads;
// each thread then scores one prior from LDS.  Kept flags are compacted with a
// wave ballot + popcount and a 4-entry cross-wave prefix, so the output order is
// the prior order.
__global__ __launch_bounds__(256) void ssd_detect_kernel(DetectParams p) {
  extern __shared__ float slab[];  // 256 * classes
  __shared__ int wave_count[4];
  __shared__ int base_shared;
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const float* logits = p.logits + (long)b * p.priors * p.classes;
  int base = 0;
  for (int start = 0; start < p.priors; start += 256) {
    const int rows = min(256, p.priors - start);
    const int count = rows * p.classes;
    const float* src = logits + (long)start * p.classes;
    for (int i = tid; i < count; i += 256) slab[i] = src[i];
    __syncthreads();

    const int prior = start + tid;
    bool keep = false;
    int max_id = 0;
    float max_prob = 0.f;
    float4 box = make_float4(0.f, 0.f, 0.f, 0.f);
    if (tid < rows) {
      const float* l = slab + tid * p.classes;
      float total_sum = exp_cr(l[0]);
      for (int j = 1; j < p.classes; ++j) {
        const float e = exp_cr(l[j]);
        total_sum += e;
        if (max_prob < e) {
          max_prob = e;
          max_id = j;
        }
      }
      const long at = (long)b * p.priors + prior;
      if (p.pred != nullptr) {
        box = decode_one(p.pred[at], p.anchors[b * p.anchor_stride_vec + prior], p.v0, p.v1,
                         p.v2, p.v3);
        if (p.boxes != nullptr) p.boxes[at] = box;
      } else {
        box = p.boxes[at];
      }
      max_prob = max_prob / total_sum;
      keep = max_prob > p.threshold;
    }
    const unsigned long long ballot = __ballot(keep);
    const int before = __popcll(ballot & ((1ull << lane) - 1ull));
    if (lane == 0) wave_count[wave] = __popcll(ballot);
    __syncthreads();
    int wave_base = 0;
    for (int wv = 0; wv < wave; ++wv) wave_base += wave_count[wv];
    if (keep) {
      const long slot = (long)b * p.priors + base + wave_base + before;
      const float xmin = box.x * p.image_w;
      const float ymin = box.y * p.image_h;
      const float xmax = box.z * p.image_w;
      const float ymax = box.w * p.image_h;
      if (p.kept_prior) p.kept_prior[slot] = prior;
      if (p.kept_class) p.kept_class[slot] = max_id;
      if (p.kept_score) p.kept_score[slot] = max_prob;
      if (p.kept_box) p.kept_box[slot] = make_float4(xmin, ymin, xmax, ymax);
      if (p.kept_rect)
        p.kept_rect[slot] = make_int4((int)xmin, (int)ymin, (int)(xmax - xmin), (int)(ymax - ymin));
    }
    if (tid == 0) base_shared = base + wave_count[0] + wave_count[1] + wave_count[2] + wave_count[3];
    __syncthreads();
    base = base_shared;
  }
  if (tid == 0) p.kept_count[b] = base;
}

// Two-kernel form of the same computation, used when every kept_* output is given:
// ssd_score_kernel spreads the per-prior work over (chunks x images) workgroups and
// leaves its results UNCOMPACTED in the kept_* arrays at the prior's own slot (prior
// index, or -1 when the prior is dropped); ssd_compact_kernel then packs each
// image's survivors to the front in place, in prior order.  A slot is only ever
// overwritten by an entry that came from the same or a later slot, after the round
// holding it has been read.
constexpr int kScorePriors = 64;  // priors per workgroup of ssd_score_kernel

__global__ __launch_bounds__(256) void ssd_score_kernel(DetectParams p) {
  // Four threads share a prior: each evaluates every fourth exponential (the costly
  // part) into LDS, then one of them makes the reference's sequential pass over the
  // row (sum in class order, strict-greater maximum), so the arithmetic and its order
  // are those of the single-thread form.
  extern __shared__ float slab[];  // logits, overwritten in place by their exponentials
  const int b = blockIdx.y;
  const int start = blockIdx.x * kScorePriors;
  const int tid = threadIdx.x;
  const int rows = min(kScorePriors, p.priors - start);
  const int count = rows * p.classes;
  const float* src = p.logits + ((long)b * p.priors + start) * p.classes;
  for (int i = tid; i < count; i += 256) slab[i] = src[i];
  __syncthreads();
  {
    const int pl = tid >> 2, q = tid & 3;
    if (pl < rows) {
      float* l = slab + pl * p.classes;
      for (int j = q; j < p.classes; j += 4) l[j] = exp_cr(l[j]);
    }
  }
  __syncthreads();
  if (tid >= rows) return;
  const int prior = start + tid;
  const float* e = slab + tid * p.classes;
  float total_sum = e[0];
  int max_id = 0;
  float max_prob = 0.f;
  for (int j = 1; j < p.classes; ++j) {
    const float ej = e[j];
    total_sum += ej;
    if (max_prob < ej) {
      max_prob = ej;
      max_id = j;
    }
  }
  const long at = (long)b * p.priors + prior;
  float4 box;
  if (p.pred != nullptr) {
    box = decode_one(p.pred[at], p.anchors[b * p.anchor_stride_vec + prior], p.v0, p.v1, p.v2, p.v3);
    if (p.boxes != nullptr) p.boxes[at] = box;
  } else {
    box = p.boxes[at];
  }
  max_prob = max_prob / total_sum;
  const bool keep = max_prob > p.threshold;
  const float xmin = box.x * p.image_w;
  const float ymin = box.y * p.image_h;
  const float xmax = box.z * p.image_w;
  const float ymax = box.w * p.image_h;
  p.kept_prior[at] = keep ? prior : -1;
  p.kept_class[at] = max_id;
  p.kept_score[at] = max_prob;
  p.kept_box[at] = make_float4(xmin, ymin, xmax, ymax);
  p.kept_rect[at] = make_int4((int)xmin, (int)ymin, (int)(xmax - xmin), (int)(ymax - ymin));
}

constexpr int kCompactThreads = 1024;
constexpr int kCompactWaves = kCompactThreads / 64;
constexpr int kCompactSlots = 2;  // entries per thread and round

__global__ __launch_bounds__(kCompactThreads) void ssd_compact_kernel(DetectParams p) {
  // A round covers kCompactThreads * kCompactSlots consecutive slots (all 1917 priors
  // of an SSD300 image in one).  Every entry of the round is read into registers with
  // all loads in flight, a barrier separates the reads from the writes, and a slot is
  // only ever overwritten by an entry from the same or a later slot, so the pass can
  // work in place.
  __shared__ int wave_count[kCompactSlots][kCompactWaves];
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const long row0 = (long)b * p.priors;
  int base = 0;
  for (int start = 0; start < p.priors; start += kCompactThreads * kCompactSlots) {
    int kept[kCompactSlots], cls[kCompactSlots], before[kCompactSlots];
    float score[kCompactSlots];
    float4 box[kCompactSlots];
    int4 rect[kCompactSlots];
#pragma unroll
    for (int u = 0; u < kCompactSlots; ++u) {
      const int prior = start + u * kCompactThreads + tid;
      kept[u] = prior < p.priors ? p.kept_prior[row0 + prior] : -1;
    }
#pragma unroll
    for (int u = 0; u < kCompactSlots; ++u) {
      const int prior = start + u * kCompactThreads + tid;
      cls[u] = 0;
      score[u] = 0.f;
      box[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      rect[u] = make_int4(0, 0, 0, 0);
      if (kept[u] >= 0) {
        cls[u] = p.kept_class[row0 + prior];
        score[u] = p.kept_score[row0 + prior];
        box[u] = p.kept_box[row0 + prior];
        rect[u] = p.kept_rect[row0 + prior];
      }
      const unsigned long long ballot = __ballot(kept[u] >= 0);
      before[u] = __popcll(ballot & ((1ull << lane) - 1ull));
      if (lane == 0) wave_count[u][wave] = __popcll(ballot);
    }
    __syncthreads();  // every read of this round is done; wave counts are visible
    int round_total = 0;
#pragma unroll
    for (int u = 0; u < kCompactSlots; ++u) {
      int slot = base + round_total + before[u];
#pragma unroll
      for (int wv = 0; wv < kCompactWaves; ++wv) {
        const int cnt = wave_count[u][wv];
        if (wv < wave) slot += cnt;
        round_total += cnt;
      }
      if (kept[u] >= 0) {
        p.kept_prior[row0 + slot] = kept[u];
        p.kept_class[row0 + slot] = cls[u];
        p.kept_score[row0 + slot] = score[u];
        p.kept_box[row0 + slot] = box[u];
        p.kept_rect[row0 + slot] = rect[u];
      }
    }
    base += round_total;
    __syncthreads();  // wave_count is rewritten by the next round
  }
  if (tid == 0) p.kept_count[b] = base;
}

// Top-k by score and the reference's NMS for one image per workgroup
// (Detector::GetTopK + Detector::NMS, detector.cc:114-148; iou, common.cc:57-77).
//   order : score descending; equal scores keep their order in the kept list
//           (ascending prior index), which is what a stable sort gives
//   NMS   : entry j is dropped if ANY earlier entry i of the top-k list has
//           iou(i, j) > threshold, whether or not i was itself dropped
// IoU is evaluated on the integer rectangles in fp32, operation by operation as the
// host does (no FMA contraction), so kept sets are bit-identical.
#pragma clang fp contract(off)
__device__ __forceinline__ float corner_iou(const float4& a, const float4& b) {
  // a, b = (xmin, ymin, xmax, ymax), the int -> float conversions iou() starts with
  const float w = fmaxf(0.0f, fminf(a.z, b.z) - fmaxf(a.x, b.x));
  const float h = fmaxf(0.0f, fminf(a.w, b.w) - fmaxf(a.y, b.y));
  const float i = w * h;
  if (i == 0.0f) return 0.0f;  // disjoint: the host gets 0 / u or its u <= 0 case, both 0
  const float u = (a.z - a.x) * (a.w - a.y) + (b.z - b.x) * (b.w - b.y) - i;
  if (u <= 0.0f) return 0.0f;
  return i / u;
}

struct NmsParams {
  const int* kept_count;
  const int* kept_prior;
  const int* kept_class;
  const float* kept_score;
  const float4* kept_box;
  const int4* kept_rect;
  int stride, topk;
  float threshold;
  int* out_count;
  int* out_prior;
  int* out_class;
  float* out_score;
  float4* out_box;
  int4* out_rect;
};

// Score bits mapped so that unsigned order equals float order (negative values too).
__device__ __forceinline__ unsigned ordered_bits(float v) {
  const unsigned b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// Steps of the kernel, one workgroup of 1024 threads per image with n kept entries:
//   1. radix select (four 8-bit passes over the ordered score bits) finds the value
//      of the k-th largest score and how many entries equal to it belong to the
//      top k; of equal scores the first ones in list order are taken
//   2. ordered compaction gathers the min(n, k) selected entries in list order
//   3. their rank under (score descending, list position ascending) is counted among
//      the selected entries only, which sorts them
//   4. NMS over all pairs of the sorted list, then an ordered compaction of the
//      survivors
constexpr int kNmsThreads = 1024;
constexpr int kNmsWaves = kNmsThreads / 64;

// Exclusive prefix of `flag` over the workgroup in thread order, and the total.
// `wave_count` is LDS scratch of kNmsWaves ints; two barriers.
__device__ __forceinline__ int block_rank(bool flag, int* wave_count, int lane, int wave, int* total) {
  const unsigned long long ballot = __ballot(flag);
  if (lane == 0) wave_count[wave] = __popcll(ballot);
  __syncthreads();
  int before = __popcll(ballot & ((1ull << lane) - 1ull));
  int sum = 0;
#pragma unroll
  for (int wv = 0; wv < kNmsWaves; ++wv) {
    const int cnt = wave_count[wv];
    if (wv < wave) before += cnt;
    sum += cnt;
  }
  __syncthreads();  // wave_count may be rewritten after this
  *total = sum;
  return before;
}

//
// SPARSE: the lists are not compacted (ogle_hip_ssd_detect without kept_count_dev): all
// `stride` slots of an image are looked at and a slot with kept_prior < 0 is empty.  An
// empty slot gets key 0, which no kept score has (scores that passed `> threshold` are
// not negative, and the key of +0 is 0x80000000), so it is never selected.
template <bool SPARSE>
__global__ __launch_bounds__(kNmsThreads) void ssd_topk_nms_kernel(NmsParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char nms_lds[];
  // keys[stride] | cand_key[topk] | cand_idx[topk] | sel[topk] | frect[topk] |
  // hist[256] | misc[kNmsWaves + 4]     (topk and stride rounded up to 4)
  const int tpad = (p.topk + 3) & ~3;
  unsigned* keys = reinterpret_cast<unsigned*>(nms_lds);
  unsigned* cand_key = keys + ((p.stride + 3) & ~3);
  int* cand_idx = reinterpret_cast<int*>(cand_key + tpad);
  int* sel = cand_idx + tpad;
  float4* frects = reinterpret_cast<float4*>(sel + tpad);
  int* hist = reinterpret_cast<int*>(frects + tpad);
  int* misc = hist + 256;  // [0..kNmsWaves) wave counts, then the chosen digit and the count above it

  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const long row0 = (long)b * p.stride;
  int n;   // slots looked at
  int nv;  // entries among them
  if constexpr (SPARSE) {
    n = p.stride;
    if (tid == 0) misc[kNmsWaves + 2] = 0;
    int mine = 0;
    for (int i = tid; i < n; i += kNmsThreads) {
      const bool live = p.kept_prior[row0 + i] >= 0;
      keys[i] = live ? ordered_bits(p.kept_score[row0 + i]) : 0u;
      mine += live ? 1 : 0;
    }
    __syncthreads();
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) mine += __shfl_xor(mine, d, 64);
    if (lane == 0 && mine > 0) atomicAdd(&misc[kNmsWaves + 2], mine);
    __syncthreads();
    nv = misc[kNmsWaves + 2];
  } else {
    n = p.kept_count[b];
    n = n < 0 ? 0 : (n > p.stride ? p.stride : n);
    nv = n;
    for (int i = tid; i < n; i += kNmsThreads) keys[i] = ordered_bits(p.kept_score[row0 + i]);
    __syncthreads();
  }

  // 1. the k-th largest key
  const int m = nv < p.topk ? nv : p.topk;
  unsigned prefix = 0, mask = 0;
  int remaining = m;  // how many of the entries matching `prefix` are still wanted
  if (nv > p.topk) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int shift = 24; shift >= 0; shift -= 8) {
      for (int i = tid; i < n; i += kNmsThreads) {
        const unsigned k = keys[i];
        // (empty slots stay out: they would all hit one counter, and cannot be chosen)
        if ((!SPARSE || k != 0u) && (k & mask) == prefix) atomicAdd(&hist[(k >> shift) & 255u], 1);
      }
      __syncthreads();
      // thread t < 256: entries whose digit is above t, and at or above t (suffix sums
      // of the histogram: a shuffle scan inside each wave plus the totals of later waves);
      // it also clears its counter for the next pass
      const int mine = tid < 256 ? hist[tid] : 0;
      if (tid < 256) hist[tid] = 0;
      int sfx = mine;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_down(sfx, d, 64);
        if (lane + d < 64) sfx += v;
      }
      if (lane == 0 && wave < 4) misc[wave] = sfx;
      __syncthreads();
      if (tid < 256) {
        int at_or_above = sfx;
        for (int wv = wave + 1; wv < 4; ++wv) at_or_above += misc[wv];
        const int above = at_or_above - mine;
        if (above < remaining && remaining <= at_or_above) {
          misc[kNmsWaves] = tid;
          misc[kNmsWaves + 1] = above;
        }
      }
      __syncthreads();
      // (the chosen digit is next written two barriers from here, the wave totals one)
      prefix |= (unsigned)misc[kNmsWaves] << shift;
      mask |= 255u << shift;
      remaining -= misc[kNmsWaves + 1];
    }
    __syncthreads();  // misc is reused by the compaction
  }
  // now: take every key above `prefix`, and the first `remaining` equal to it
  // (nv <= topk: every entry is taken)

  // 2. ordered compaction of the selected entries.  A thread takes a contiguous run of slots
  // and counts, in one packed word, its entries above the k-th key and its entries equal to
  // it; one scan over the workgroup gives both counts for everything before the run, and an
  // entry's place follows from them: (above before it) + min(equal before it, remaining).
  {
    const int per = (n + kNmsThreads - 1) / kNmsThreads;
    const int first = tid * per;
    unsigned mine = 0;  // above | equal << 16  (n < 65536: the keys fit in LDS)
    for (int e = 0; e < per; ++e) {
      const int i = first + e;
      const unsigned k = i < n ? keys[i] : 0u;
      const bool live = i < n && (!SPARSE || k != 0u);
      if (live && (nv <= p.topk || k > prefix)) mine += 1u;
      if (live && nv > p.topk && k == prefix) mine += 65536u;
    }
    unsigned incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const unsigned v = __shfl_up(incl, d, 64);
      if (lane >= d) incl += v;
    }
    unsigned* wave_total = reinterpret_cast<unsigned*>(misc);
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    unsigned before = incl - mine;
    for (int wv = 0; wv < wave; ++wv) before += wave_total[wv];
    int above = (int)(before & 0xffffu), equal = (int)(before >> 16);
    for (int e = 0; e < per; ++e) {
      const int i = first + e;
      const unsigned k = i < n ? keys[i] : 0u;
      const bool live = i < n && (!SPARSE || k != 0u);
      const bool gt = live && (nv <= p.topk || k > prefix);
      const bool eq = live && nv > p.topk && k == prefix;
      if (gt || (eq && equal < remaining)) {
        const int at = above + (equal < remaining ? equal : remaining);
        cand_key[at] = k;
        cand_idx[at] = i;
      }
      above += gt ? 1 : 0;
      equal += eq ? 1 : 0;
    }
  }
  for (int r = m + tid; r < ((m + 3) & ~3); r += kNmsThreads) cand_key[r] = 0u;  // padding ranks last
  __syncthreads();

  // 3. thread r owns selected entry r (topk <= the thread count): its record is
  // requested now, and its rank among the selected entries (they are in list order,
  // so position breaks ties) is counted while the loads are in flight
  const int mpad = (m + 3) & ~3;
  const bool owner = tid < m;
  int my_prior = 0, my_class = 0, my_rank = 0;
  float my_score = 0.f;
  float4 my_box = make_float4(0.f, 0.f, 0.f, 0.f);
  int4 my_rect = make_int4(0, 0, 0, 0);
  if (owner) {
    const long src = row0 + cand_idx[tid];
    my_rect = p.kept_rect[src];
    my_prior = p.kept_prior[src];
    my_class = p.kept_class[src];
    my_score = p.kept_score[src];
    if (p.kept_box != nullptr) my_box = p.kept_box[src];
    const unsigned kr = cand_key[tid];
    for (int j = 0; j < mpad; j += 4) {
      const uint4 v = *reinterpret_cast<const uint4*>(cand_key + j);
      my_rank += (v.x > kr || (v.x == kr && j + 0 < tid)) ? 1 : 0;
      my_rank += (v.y > kr || (v.y == kr && j + 1 < tid)) ? 1 : 0;
      my_rank += (v.z > kr || (v.z == kr && j + 2 < tid)) ? 1 : 0;
      my_rank += (v.w > kr || (v.w == kr && j + 3 < tid)) ? 1 : 0;
    }
    // corners as the host's iou() forms them: integer sums converted to float
    frects[my_rank] = make_float4((float)my_rect.x, (float)my_rect.y, (float)(my_rect.x + my_rect.z),
                                  (float)(my_rect.y + my_rect.w));
  }
  int* dropped = sel;  // [rank] -> 1 if suppressed
  for (int r = tid; r < m; r += kNmsThreads) dropped[r] = 0;
  __syncthreads();

  // 4. NMS: all (i, j) pairs with i < j are spread over the workgroup; a pair that
  // overlaps by more than the threshold marks j (every writer stores the same value)
  if (m > 1) {
    // Only the pairs with i < j are visited: they are laid out as rows of equal length (row a
    // holds the pairs (a, j > a) and fills up with those of the row that mirrors it), and a
    // thread steps through them by the thread count without dividing.
    const bool odd = (m & 1) != 0;
    const int len = odd ? m : m - 1;
    const int rows = odd ? (m - 1) / 2 : m / 2;
    const int step_a = kNmsThreads / len, step_b = kNmsThreads - step_a * len;
    int a = tid / len, b = tid - a * len;
    for (; a < rows; a += step_a, b += step_b) {
      if (b >= len) {
        b -= len;
        ++a;
        if (a >= rows) break;
      }
      int i, j;
      if (odd) {
        i = b > a ? a : m - 2 - a;
        j = b > a ? b : m - 1 - b;
      } else {
        i = b >= a ? a : m - 1 - a;
        j = b >= a ? b + 1 : m - 1 - b;
      }
      if (corner_iou(frects[i], frects[j]) > p.threshold) dropped[j] = 1;
    }
  }
  __syncthreads();

  // output position of every surviving rank (ordered compaction over the ranks), then
  // each owner writes its record from registers
  int* out_pos = cand_idx;  // the candidate list is no longer needed
  int total;
  {
    const bool keep = tid < m && dropped[tid] == 0;
    const int before = block_rank(keep, misc, lane, wave, &total);
    if (tid < m) out_pos[tid] = keep ? before : -1;
  }
  __syncthreads();
  if (owner) {
    const int o = out_pos[my_rank];
    if (o >= 0) {
      const long dst = (long)b * p.topk + o;
      p.out_prior[dst] = my_prior;
      p.out_class[dst] = my_class;
      p.out_score[dst] = my_score;
      if (p.out_box != nullptr) p.out_box[dst] = my_box;
      p.out_rect[dst] = my_rect;
    }
  }
  if (tid == 0) p.out_count[b] = total;
}

}  // namespace

size_t topk_nms_lds_bytes(int stride, int topk) {
  const size_t tpad = (size_t)((topk + 3) & ~3);
  return 4 * (size_t)((stride + 3) & ~3) + 4 * 3 * tpad + sizeof(float4) * tpad +
         4 * (256 + kNmsWaves + 4);
}

int32_t launch_topk_nms(const OgleNmsArgs& a, hipStream_t s) {
  if (a.batch == 0) return OGLE_OK;
  NmsParams p{};
  p.kept_count = a.kept_count_dev;
  p.kept_prior = a.kept_prior_dev;
  p.kept_class = a.kept_class_dev;
  p.kept_score = a.kept_score_dev;
  p.kept_box = reinterpret_cast<const float4*>(a.kept_box_dev);
  p.kept_rect = reinterpret_cast<const int4*>(a.kept_rect_dev);
  p.stride = a.stride;
  p.topk = a.topk;
  p.threshold = a.nms_threshold;
  p.out_count = a.final_count_dev;
  p.out_prior = a.final_prior_dev;
  p.out_class = a.final_class_dev;
  p.out_score = a.final_score_dev;
  p.out_box = reinterpret_cast<float4*>(a.final_box_dev);
  p.out_rect = reinterpret_cast<int4*>(a.final_rect_dev);
  if (a.kept_count_dev == nullptr) {
    launch(ssd_topk_nms_kernel<true>, dim3((unsigned)a.batch), dim3(kNmsThreads),
                       topk_nms_lds_bytes(a.stride, a.topk), s, p);
  } else {
    launch(ssd_topk_nms_kernel<false>, dim3((unsigned)a.batch), dim3(kNmsThreads),
                       topk_nms_lds_bytes(a.stride, a.topk), s, p);
  }
  return check_launch("ssd_topk_nms_kernel");
}

int32_t launch_decode(const OgleDecodeArgs& a, hipStream_t s) {
  const long total = (long)a.batch * a.priors;
  if (total == 0) return OGLE_OK;
  long blocks = (total + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  launch(ssd_decode_kernel, dim3((unsigned)blocks), dim3(256), 0, s,
                     reinterpret_cast<const float4*>(a.prediction_dev),
                     reinterpret_cast<const float4*>(a.anchors_dev),
                     reinterpret_cast<float4*>(a.boxes_dev), a.batch, a.priors,
                     (long)(a.anchors_batch_stride / 4), a.variances[0], a.variances[1],
                     a.variances[2], a.variances[3]);
  return check_launch("ssd_decode_kernel");
}

int32_t launch_detect(const OgleDetectArgs& a, hipStream_t s) {
  if (a.batch == 0) return OGLE_OK;
  DetectParams p{};
  p.logits = a.logits_dev;
  p.pred = reinterpret_cast<const float4*>(a.prediction_dev);
  p.anchors = reinterpret_cast<const float4*>(a.anchors_dev);
  p.boxes = reinterpret_cast<float4*>(a.boxes_dev);
  p.batch = a.batch; p.priors = a.priors; p.classes = a.classes;
  p.anchor_stride_vec = (long)(a.anchors_batch_stride / 4);
  p.v0 = a.variances[0]; p.v1 = a.variances[1]; p.v2 = a.variances[2]; p.v3 = a.variances[3];
  p.threshold = a.score_threshold; p.image_w = a.image_width; p.image_h = a.image_height;
  p.kept_count = a.kept_count_dev; p.kept_prior = a.kept_prior_dev;
  p.kept_class = a.kept_class_dev; p.kept_score = a.kept_score_dev;
  p.kept_box = reinterpret_cast<float4*>(a.kept_box_dev);
  p.kept_rect = reinterpret_cast<int4*>(a.kept_rect_dev);
  const size_t lds = sizeof(float) * 256 * (size_t)a.classes;
  const bool all_outputs = p.kept_prior && p.kept_class && p.kept_score && p.kept_box && p.kept_rect;
  const bool sparse = p.kept_count == nullptr;  // validated: all outputs given, batch <= 65535
  if (sparse && a.priors == 0) return OGLE_OK;
  if (sparse || (all_outputs && a.priors > 256 && a.batch <= 65535)) {
    launch(ssd_score_kernel,
                       dim3((unsigned)((a.priors + kScorePriors - 1) / kScorePriors), (unsigned)a.batch),
                       dim3(256), sizeof(float) * kScorePriors * (size_t)a.classes, s, p);
    const int32_t st = check_launch("ssd_score_kernel");
    if (st != OGLE_OK || sparse) return st;
    launch(ssd_compact_kernel, dim3((unsigned)a.batch), dim3(kCompactThreads), 0, s, p);
    return check_launch("ssd_compact_kernel");
  }
  launch(ssd_detect_kernel, dim3((unsigned)a.batch), dim3(256), lds, s, p);
  return check_launch("ssd_detect_kernel");
}

int32_t launch_expf(const float* x, float* y, int64_t n, hipStream_t s) {
  if (n == 0) return OGLE_OK;
  long blocks = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  launch(expf_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, y, (long)n);
  return check_launch("expf_kernel");
}

}  // namespace ogle
