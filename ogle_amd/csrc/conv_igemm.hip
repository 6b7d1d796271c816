// Dense convolution (group 1) as an implicit GEMM on the MFMA units.
//
//   Y[m, o] = act( bias[o] + sum_{tap, c} X[row(m) + tap, c] * W[o, tap, c] )
//
// with m = (image, oy, ox) flattened, K = taps * C.  Both operands are
// K-contiguous in memory: X is NHWC (a pixel's channels are contiguous) and W is
// packed OHWI (an output channel's taps*channels are contiguous), so both tiles
// are fetched as 16-byte vectors along K and the pointwise 1x1 convolution is the
// special case with one tap and no gather (conv2d_pw.glsl:35-91); the KxK form
// follows conv2d.glsl:29-92 (taps outside the image contribute zero).
//
// Tiling.  A workgroup of 4 waves (256 threads) owns a BM x BN output tile and
// walks K in slabs of ROWB bytes per row.  Slabs are staged global -> registers
// -> LDS (double buffered, one barrier per slab) with the next slab's global
// loads in flight while the current one is multiplied.  LDS rows are padded by
// 16 bytes so the 16-byte-per-lane operand reads are bank-conflict free.
//
// MFMA mapping (64-wide waves).  fp32 uses v_mfma_f32_32x32x2_f32: lane l
// supplies A[l%32][l/32] and B[l/32][l%32].  Since the contraction sums over k
// in any order, a lane reads four consecutive k of its row with one 16-byte LDS
// read (lanes 0-31 take k 0..3 of an 8-wide group, lanes 32-63 take k 4..7) and
// issues four MFMAs, one per element.  fp16 storage uses
// v_mfma_f32_32x32x16_f16: a lane's 16 bytes are the 8 halves the instruction
// wants (k = 8*(l/32)..+7).  Accumulation is fp32 in both cases.
//
// Result layout of a 32x32 block: register r of lane l holds
// row 8*(r/4) + 4*(l/32) + r%4, column l%32, so a store instruction writes two
// 128-byte runs of one output pixel's channels.
//
// A tile that is 16 columns wide (at most 16 output channels) is built from 16x16
// blocks instead: v_mfma_f32_16x16x4_f32 (lane l supplies A[l%16][l/16], four lane
// groups take k 0..3, 4..7, 8..11, 12..15 of a 16-wide group and issue four MFMAs)
// or v_mfma_f32_16x16x32_f16; register r of lane l is row 4*(l/16) + r, column l%16.
#include <mutex>
#include <vector>

#include "common.h"

namespace ogle {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));

struct ConvGeom {
  int n, h, w, c;
  int oh, ow, o;
  int k, stride, pad, dil;
  int m_total;   // n*oh*ow
  int cchunks;   // K slabs per tap
  int ktiles;    // taps * cchunks
  unsigned x_bytes;  // size of the input tensor (buffer-load range)
  unsigned w_bytes;  // size of the packed filter
  long oimg;         // elements between the outputs of consecutive images; 0: dense
};

// Element offset of output row `row` (= (image, oy, ox) flattened) whose channels are
// `pitch` apart per row: dense, or with a gap after every image's oh * ow rows.
__device__ __forceinline__ long out_row_offset(const ConvGeom& g, int row, int pitch) {
  if (g.oimg == 0) return (long)row * pitch;
  const int hw = g.oh * g.ow;
  const int b = row / hw;
  return (long)b * g.oimg + (long)(row - b * hw) * pitch;
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Offset that is out of range for every operand (operands are kept below 2 GiB), so
// a buffer load at it returns zeros: this is how padding taps, rows past the end of
// the problem and the K tail are zero filled without a branch.
constexpr unsigned kOutOfRange = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

typedef float floatx4v __attribute__((ext_vector_type(4)));

// MFMA step on a TS x TS block of outputs (the wave-split kernel's tile; the LDS-tiled
// kernel's block when its tile is 16 columns wide).  `a` / `b` are the 16 bytes
// the lane loaded; lanes are grouped by q = lane / TS.
//   TS 32: q in {0,1};   fp32 4 x 32x32x2 (k = 4q + s), fp16 1 x 32x32x16 (k = 8q..)
//   TS 16: q in {0..3};  fp32 4 x 16x16x4 (k = 4q + s), fp16 1 x 16x16x32 (k = 8q..)
template <typename T, int TS>
struct WaveMma;
template <>
struct WaveMma<float, 32> {
  typedef floatx16 Acc;
  static constexpr int REGS = 16;
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, Acc& acc) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[s]), __uint_as_float(b[s]), acc, 0, 0, 0);
  }
};
template <>
struct WaveMma<__half, 32> {
  typedef floatx16 Acc;
  static constexpr int REGS = 16;
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, Acc& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a),
                                                 __builtin_bit_cast(halfx8, b), acc, 0, 0, 0);
  }
};
template <>
struct WaveMma<float, 16> {
  typedef floatx4v Acc;
  static constexpr int REGS = 4;
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, Acc& acc) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a[s]), __uint_as_float(b[s]), acc, 0, 0, 0);
  }
};
template <>
struct WaveMma<__half, 16> {
  typedef floatx4v Acc;
  static constexpr int REGS = 4;
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, Acc& acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, a),
                                                 __builtin_bit_cast(halfx8, b), acc, 0, 0, 0);
  }
};

// One workgroup's share of one convolution: output tile / K range number `bid` of
// the problem.  Shared by the single-problem kernel and the grouped kernel.
// LDS bytes of one workgroup: two K-slab buffers of BM + BN padded rows.
template <int BM, int BN, int ROWB>
constexpr int igemm_lds_bytes() {
  return 2 * (BM + BN) * (ROWB + 16);
}

template <typename T, int BM, int BN, int WM, int WN, int ROWB, bool PW>
__device__ __forceinline__ void igemm_tile(
    unsigned char* __restrict__ lds, const ConvGeom& g, const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ bias, T* __restrict__ y, T* __restrict__ y2, int o1,
    const Epilogue& ep, int tiles_n, int tiles, float* __restrict__ partial,
    int slabs_per_split, int splits, int bid) {
  static_assert(WM * WN == 4, "four waves per workgroup");
  constexpr int WTM = BM / WM, WTN = BN / WN;
  // MFMA block: 32x32 outputs, or 16x16 (v_mfma_f32_16x16x4_f32 / 16x16x32_f16) for a tile
  // that is only 16 columns wide (a convolution with at most 16 output channels: in a
  // 32-wide block more than half of the MFMA work would be padding)
  constexpr int MB = WTN % 32 == 0 ? 32 : 16;
  constexpr int TM = WTM / MB, TN = WTN / MB;
  static_assert(TM >= 1 && TN >= 1 && WTM % MB == 0 && WTN % MB == 0, "wave tile in whole MFMA blocks");
  typedef typename WaveMma<T, MB>::Acc Acc;
  constexpr int REGS = WaveMma<T, MB>::REGS;
  constexpr int VPR = ROWB / 16;       // 16-byte vectors per row per slab
  constexpr int RPP = 256 / VPR;       // rows one pass of the workgroup loads
  constexpr int AP = (BM + RPP - 1) / RPP, BP = (BN + RPP - 1) / RPP;
  constexpr bool A_PART = BM % RPP != 0, B_PART = BN % RPP != 0;  // last pass partly idle
  // LDS rows.  A row is exactly its slab bytes and its 16-byte K groups are permuted by a
  // function of the row: (row >> 1) & 7 for 128-byte rows; for 64-byte rows (row >> 2) & 3
  // under 32x32 MFMA blocks and 2 * ((row >> 2) & 1) under 16x16 blocks.  That keeps both the
  // operand reads and the staging writes free of bank conflicts (a 16-byte LDS access is
  // served 16 lanes per cycle: those with the same lane / 32 and the same parity of
  // (lane >> 2) & 7; they must fall into 16 different 16-byte columns of a 256-byte window;
  // found by exhaustive search over XOR functions of the row bits against that model,
  // confirmed by SQ_LDS_BANK_CONFLICT: 1.58 M -> 0.05 M cycles per launch of a
  // 19x19x512 -> 512 pointwise layer at batch 16; rows padded by 16 bytes, as before, cost the
  // writes three times and the 16x16 reads twice the conflict-free cycles).  Other slab
  // widths: rows padded by 16 bytes.
  constexpr bool SWZ = ROWB == 64 || ROWB == 128;
  constexpr int LROW = SWZ ? ROWB : ROWB + 16;   // LDS row pitch, bytes
  auto row_perm = [](int row) {
    return ROWB == 128 ? (row >> 1) & 7 : MB == 32 ? (row >> 2) & 3 : ((row >> 2) & 1) << 1;
  };
  constexpr int ESZ = (int)sizeof(T);
  constexpr int CHUNKB = (64 / MB) * 16;  // bytes of a row one MFMA step consumes (64 / MB lane groups x 16)
  constexpr int CHUNKS = ROWB / CHUNKB;
  static_assert(CHUNKS >= 1, "a K slab holds at least one MFMA step");
  constexpr int STAGE = (BM + BN) * (ROWB + 16);  // one buffer: A rows then B rows

  static_assert(2 * STAGE == igemm_lds_bytes<BM, BN, ROWB>(), "LDS size");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WN, wave_n = wave % WN;

  // Work assignment.  Workgroups are dealt to the 8 XCDs by linear id modulo 8 and
  // every XCD has a private L2, so the (tile, split) pairs are laid out such that
  // tiles sharing a band of A rows run on one XCD and, when K is split, an XCD owns
  // a fixed subset of the K ranges: the filter and input slabs of one K range are
  // then fetched into one L2 only instead of all eight.
  // When K is split and the input is the larger operand (a 3x3 head on a big map), the
  // other layout is used instead (splits < 0 marks it): tile rows are dealt to the XCDs and
  // all K ranges of a tile row run on the same XCD, so each band of input rows (with the
  // halo its taps share) is fetched into one L2 only, and the filter into all eight.
  int pid, split;
  if (splits < 0) {
    splits = -splits;
    const int xcd = bid & 7, j = bid >> 3;
    const int per_row = tiles_n * splits;
    const int r = (j / per_row) * 8 + xcd;
    const int rem = j % per_row;
    pid = r * tiles_n + rem / splits;
    split = rem % splits;
    if (pid >= tiles) return;
  } else {
    const int xcd = bid & 7, j = bid >> 3;
    if (splits == 1) {
      // tile row r (the tiles_n tiles that share one band of A rows) goes to XCD
      // r % 8, so all XCDs advance through memory together
      const int r = (j / tiles_n) * 8 + xcd;
      pid = r * tiles_n + j % tiles_n;
      split = 0;
    } else if (splits >= 8 && (splits & 7) == 0) {
      const int zs = splits >> 3;
      pid = j / zs;
      split = xcd + 8 * (j - pid * zs);
    } else if (splits == 2 || splits == 4) {
      const int xpz = 8 / splits;
      split = xcd % splits;
      pid = j * xpz + xcd / splits;
    } else {                       // any other count: the splits of a tile are neighbours
      pid = bid / splits;
      split = bid - pid * splits;
    }
    if (pid >= tiles) return;
  }
  const int tile_n = pid % tiles_n;
  const int tile_m = pid / tiles_n;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * BN;

  const int vcol = tid % VPR;   // which 16-byte vector of the slab row
  const int vrow = tid / VPR;   // row within a pass

  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x, g.x_bytes);
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(w, g.w_bytes);

  // Per-pass source rows of this thread, as byte offsets into the operands.
  unsigned a_base[AP];  // PW: row offset; KxK: offset of the image the row lies in
  int a_iy[AP], a_ix[AP];
#pragma unroll
  for (int p = 0; p < AP; ++p) {
    const int m = m0 + p * RPP + vrow;
    const bool ok = m < g.m_total && (!A_PART || p * RPP + vrow < BM);
    if (PW) {
      a_base[p] = ok ? (unsigned)m * (unsigned)(g.c * ESZ) : kOutOfRange;
      a_iy[p] = 0;
      a_ix[p] = 0;
    } else {
      const int ox = m % g.ow;
      const int t = m / g.ow;
      const int oy = t % g.oh;
      const int b = t / g.oh;
      a_base[p] = (unsigned)b * (unsigned)(g.h * g.w * g.c * ESZ);
      // a row that does not exist fails every in-image test below
      a_iy[p] = ok ? oy * g.stride - g.pad : -0x40000000;
      a_ix[p] = ox * g.stride - g.pad;
    }
  }
  const unsigned krow_bytes = (unsigned)(g.k * g.k * g.c * ESZ);
  unsigned b_base[BP];
#pragma unroll
  for (int p = 0; p < BP; ++p) {
    const int o = n0 + p * RPP + vrow;
    const bool ok = o < g.o && (!B_PART || p * RPP + vrow < BN);
    b_base[p] = ok ? (unsigned)o * krow_bytes : kOutOfRange;
  }

  // Two register sets: slab kt+1 is already in flight in one while slab kt+2 is
  // being requested into the other, so a load has two slabs of MFMA work to land.
  u32x4 ra[2][AP], rb[2][BP];

  // Issues the global loads of the next K slab into ra / rb (no waiting) and moves
  // the load cursor on.  The cursor (slab number, its tap, channel chunk and tap
  // offsets) advances by increments: slabs are requested strictly in order, so the
  // two integer divisions that locate a slab are paid once, not per slab.
#define OGLE_LOAD_SLAB(SET)                                                                  \
  {                                                                                          \
    const int cbyte_ = l_cc * ROWB + vcol * 16;                                              \
    const bool c_ok_ = cbyte_ < g.c * ESZ && l_kt < kt_end; /* past the end: zeros */        \
    _Pragma("unroll") for (int p = 0; p < AP; ++p) {                                         \
      unsigned off_;                                                                         \
      if (PW) {                                                                              \
        off_ = c_ok_ ? a_base[p] + (unsigned)cbyte_ : kOutOfRange;                           \
      } else {                                                                               \
        const int iy_ = a_iy[p] + l_dy, ix_ = a_ix[p] + l_dx;                                \
        const bool in_ = c_ok_ && iy_ >= 0 && iy_ < g.h && ix_ >= 0 && ix_ < g.w;            \
        off_ = in_ ? a_base[p] + (unsigned)((iy_ * g.w + ix_) * g.c * ESZ + cbyte_)          \
                   : kOutOfRange;                                                            \
      }                                                                                      \
      ra[SET][p] = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)off_, 0, 0);               \
    }                                                                                        \
    _Pragma("unroll") for (int p = 0; p < BP; ++p) {                                         \
      const unsigned off_ = c_ok_ ? b_base[p] + l_tapbyte + (unsigned)cbyte_ : kOutOfRange;  \
      rb[SET][p] = __builtin_amdgcn_raw_buffer_load_b128(rw, (int)off_, 0, 0);               \
    }                                                                                        \
    ++l_kt;                                                                                  \
    if (++l_cc == g.cchunks) {                                                               \
      l_cc = 0;                                                                              \
      l_tapbyte += (unsigned)(g.c * ESZ);                                                    \
      l_dx += g.dil;                                                                         \
      if (++l_kx == g.k) {                                                                   \
        l_kx = 0;                                                                            \
        l_dx = 0;                                                                            \
        l_dy += g.dil;                                                                       \
      }                                                                                      \
    }                                                                                        \
  }

  // Writes ra / rb into LDS buffer `buf`.
#define OGLE_STORE_SLAB(buf, SET)                                                            \
  {                                                                                          \
    unsigned char* base_ = lds + (buf) * STAGE + vrow * LROW +                               \
                           (SWZ ? (vcol ^ row_perm(vrow)) : vcol) * 16;                      \
    _Pragma("unroll") for (int p = 0; p < AP; ++p)                                           \
      if (!A_PART || p * RPP + vrow < BM)                                                    \
        *reinterpret_cast<u32x4*>(base_ + p * RPP * LROW) = ra[SET][p];                      \
    _Pragma("unroll") for (int p = 0; p < BP; ++p)                                           \
      if (!B_PART || p * RPP + vrow < BN)                                                    \
        *reinterpret_cast<u32x4*>(base_ + (BM + p * RPP) * LROW) = rb[SET][p];               \
  }

  Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < REGS; ++r) acc[i][j][r] = 0.f;

  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int lrow = lane % MB;  // operand row of this lane inside an MFMA block
  const int lq = lane / MB;    // its 16-byte group along K

  // Split-K: workgroup z of the grid contracts K slabs [kt_begin, kt_end) only and
  // leaves its partial sums in `partial`; a second kernel adds the splits in order.
  const int kt_begin = split * slabs_per_split;
  const int kt_end = min(g.ktiles, kt_begin + slabs_per_split);

  // One K slab from LDS buffer `buf` into the accumulators.
#define OGLE_COMPUTE_SLAB(buf)                                                               \
  {                                                                                          \
    const unsigned char* pa = lds + (buf) * STAGE + (wave_m * WTM + lrow) * LROW;            \
    const unsigned char* pb = lds + (buf) * STAGE + (BM + wave_n * WTN + lrow) * LROW;       \
    _Pragma("unroll") for (int ch = 0; ch < CHUNKS; ++ch) {                                  \
      /* this lane's 16-byte K group of the step (rows 32 apart share the permutation) */    \
      const int kof = SWZ ? (((ch * (CHUNKB / 16) + lq) ^ row_perm(lrow)) * 16)              \
                          : lq * 16 + ch * CHUNKB;                                           \
      u32x4 av[TM], bv[TN];                                                                  \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                         \
        av[i] = *reinterpret_cast<const u32x4*>(pa + i * MB * LROW + kof);                   \
      _Pragma("unroll") for (int j = 0; j < TN; ++j)                                         \
        bv[j] = *reinterpret_cast<const u32x4*>(pb + j * MB * LROW + kof);                   \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                         \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                       \
          WaveMma<T, MB>::run(av[i], bv[j], acc[i][j]);                                      \
    }                                                                                        \
  }

  // The load cursor starts at slab kt_begin.
  int l_kt = kt_begin, l_cc = kt_begin, l_kx = 0, l_dy = 0, l_dx = 0;
  unsigned l_tapbyte = 0;
  if (!PW) {
    const int tap = kt_begin / g.cchunks;
    const int ky = tap / g.k;
    l_cc = kt_begin - tap * g.cchunks;
    l_kx = tap - ky * g.k;
    l_dy = ky * g.dil;
    l_dx = l_kx * g.dil;
    l_tapbyte = (unsigned)(tap * g.c * ESZ);
  }

  // Software pipeline, unrolled by two so that the register sets and LDS buffers
  // are compile-time: while slab kt is multiplied out of one LDS buffer, slab kt+1
  // (requested one step earlier) is moved from its registers into the other buffer
  // and slab kt+2 is requested.  Requests past kt_end return zeros and are dropped.
  OGLE_LOAD_SLAB(0);
  OGLE_LOAD_SLAB(1);
  OGLE_STORE_SLAB(0, 0);
  __syncthreads();
  for (int kt = kt_begin; kt < kt_end; kt += 2) {
    // An odd slab count runs one extra all-zero slab through the second half: a
    // loop without early exits keeps the accumulators in one set of registers.
    OGLE_LOAD_SLAB(0);
    OGLE_COMPUTE_SLAB(0);
    OGLE_STORE_SLAB(1, 1);
    __syncthreads();
    OGLE_LOAD_SLAB(1);
    OGLE_COMPUTE_SLAB(1);
    OGLE_STORE_SLAB(0, 0);
    __syncthreads();
  }
#undef OGLE_COMPUTE_SLAB
#undef OGLE_LOAD_SLAB
#undef OGLE_STORE_SLAB

  // Epilogue.  Destinations: split-K partial sums go to `partial` (rows of opitch floats,
  // the channel count rounded up to 4 so that rows stay 16-byte aligned); finished outputs
  // go to y, or, with a second destination, channels [0, o1) to y (o1 per pixel) and
  // channels [o1, o) to y2 (o - o1 per pixel).  When the row pitches allow 16-byte stores
  // the accumulators go through a wave-private LDS region to be transposed from the MFMA
  // layout (a lane holds one column) into rows, so that a wave writes whole contiguous row
  // segments with 16-byte stores; bias and activation are applied on the way out.
  // Otherwise each lane stores its elements one by one (32 lanes cover 128 contiguous
  // bytes of a row).
  const int opitch = (g.o + 3) & ~3;
  const int o2 = g.o - o1;
  float* const pdst = partial != nullptr ? partial + (long)split * g.m_total * opitch : nullptr;
  if constexpr (MB == 16) {
    // 16x16 blocks: register r of lane l is row 4 * (l / 16) + r, column l % 16, so the 16
    // lanes of a group store one 64-byte run of an output row.  Partial rows are written
    // up to their padded width (the columns past the last channel hold zeros).
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wave_n * WTN + j * 16 + lrow;
      const float bv = (pdst == nullptr && bias != nullptr && col < g.o) ? bias[col] : 0.f;
      const bool second = col >= o1;
      T* const dst = second ? y2 + (col - o1) : y + col;
      const int dpitch = second ? o2 : o1;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < REGS; ++r) {
          const int row = m0 + wave_m * WTM + i * 16 + lq * 4 + r;
          if (row >= g.m_total) continue;
          if (pdst != nullptr) {
            if (col < opitch) pdst[(long)row * opitch + col] = acc[i][j][r];
          } else if (col < g.o) {
            dst[out_row_offset(g, row, dpitch)] = from_f32<T>(apply_epilogue(acc[i][j][r] + bv, ep));
          }
        }
      }
    }
    return;
  } else {
  // The staging region (reused K-loop LDS) takes JC 32-column blocks of a wave's tile at a
  // time: as many as fit, so that a row segment a wave stores is as long as possible.
  constexpr auto stage_fits = [](int jc) { return 4 * 32 * (jc * 32 + 4) * 4 <= 2 * STAGE; };
  constexpr int JC = (TN % 4 == 0 && stage_fits(4)) ? 4 : (TN % 2 == 0 && stage_fits(2)) ? 2 : 1;
  static_assert(stage_fits(JC), "epilogue staging exceeds the K-loop LDS");
  constexpr int CW = JC * 32;              // columns staged at once
  constexpr int SROW = CW + 4;             // floats per staged row (padded)
  float* const smw = reinterpret_cast<float*>(lds) + wave * 32 * SROW;
  if (pdst != nullptr || (sizeof(T) == 4 && (o1 & 3) == 0 && (o2 & 3) == 0 && (g.oimg & 3) == 0)) {
    constexpr int LPR = CW / 4;              // lanes covering one staged row
    constexpr int RPI = 64 / LPR;            // rows one store instruction covers
    const int cv = lane % LPR;
    const int rsub = lane / LPR;
#pragma unroll
    for (int j0 = 0; j0 < TN; j0 += JC) {
      const int col = n0 + wave_n * WTN + j0 * 32 + cv * 4;
      float4 bias4 = make_float4(0.f, 0.f, 0.f, 0.f);
      if (pdst == nullptr && bias != nullptr && col < g.o)
        bias4 = *reinterpret_cast<const float4*>(bias + col);
      // row pitch and first column of the destination this lane's four channels lie in
      const bool second = pdst == nullptr && col >= o1;
      const int dpitch = pdst != nullptr ? opitch : (second ? o2 : o1);
      const int dcol = second ? col - o1 : col;
      float* const dbase = pdst != nullptr ? pdst : reinterpret_cast<float*>(second ? y2 : y);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < JC; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            smw[((r >> 2) * 8 + lh * 4 + (r & 3)) * SROW + j * 32 + l32] = acc[i][j0 + j][r];
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
          const int row = it * RPI + rsub;
          float4 v = *reinterpret_cast<const float4*>(smw + row * SROW + cv * 4);
          const int grow = m0 + wave_m * WTM + i * 32 + row;
          if (grow < g.m_total && col < g.o) {
            if (pdst == nullptr) {
              v.x = apply_epilogue(v.x + bias4.x, ep);
              v.y = apply_epilogue(v.y + bias4.y, ep);
              v.z = apply_epilogue(v.z + bias4.z, ep);
              v.w = apply_epilogue(v.w + bias4.w, ep);
            }
            const long at = pdst != nullptr ? (long)grow * dpitch : out_row_offset(g, grow, dpitch);
            store_result16(dbase + at + dcol, v);
          }
        }
      }
    }
    return;
  }
  if constexpr (sizeof(T) == 2) {
    if ((g.o & 7) == 0 && y2 == nullptr && (g.oimg & 7) == 0) {
      // fp16 output: the same staging, a lane then takes eight consecutive channels
      // of a row and stores them as one 16-byte vector of halves
      constexpr int LPR = CW / 8;
      constexpr int RPI = 64 / LPR;
      const int cv = lane % LPR;
      const int rsub = lane / LPR;
#pragma unroll
      for (int j0 = 0; j0 < TN; j0 += JC) {
        const int col = n0 + wave_n * WTN + j0 * 32 + cv * 8;
        float bias8[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) bias8[q] = 0.f;
        if (bias != nullptr && col < g.o) {
          const float4 b0 = *reinterpret_cast<const float4*>(bias + col);
          const float4 b1 = *reinterpret_cast<const float4*>(bias + col + 4);
          bias8[0] = b0.x; bias8[1] = b0.y; bias8[2] = b0.z; bias8[3] = b0.w;
          bias8[4] = b1.x; bias8[5] = b1.y; bias8[6] = b1.z; bias8[7] = b1.w;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
          for (int j = 0; j < JC; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              smw[((r >> 2) * 8 + lh * 4 + (r & 3)) * SROW + j * 32 + l32] = acc[i][j0 + j][r];
#pragma unroll
          for (int it = 0; it < 32 / RPI; ++it) {
            const int row = it * RPI + rsub;
            const float4 v0 = *reinterpret_cast<const float4*>(smw + row * SROW + cv * 8);
            const float4 v1 = *reinterpret_cast<const float4*>(smw + row * SROW + cv * 8 + 4);
            const int grow = m0 + wave_m * WTM + i * 32 + row;
            if (grow < g.m_total && col < g.o) {
              const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
              uint4 packed;
              __half2* h = reinterpret_cast<__half2*>(&packed);
#pragma unroll
              for (int q = 0; q < 4; ++q)
                h[q] = __floats2half2_rn(apply_epilogue(f[2 * q] + bias8[2 * q], ep),
                                         apply_epilogue(f[2 * q + 1] + bias8[2 * q + 1], ep));
              store_result16(reinterpret_cast<__half*>(y) + out_row_offset(g, grow, g.o) + col, packed);
            }
          }
        }
      }
      return;
    }
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wave_n * WTN + j * 32 + l32;
    if (col >= g.o) continue;
    const float bv = (pdst == nullptr && bias != nullptr) ? bias[col] : 0.f;
    const bool second = col >= o1;
    T* const dst = second ? y2 + (col - o1) : y + col;
    const int dpitch = second ? o2 : o1;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int rbase = m0 + wave_m * WTM + i * 32 + lh * 4;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = rbase + (r >> 2) * 8 + (r & 3);
        if (row >= g.m_total) continue;
        if (pdst != nullptr) {
          pdst[(long)row * opitch + col] = acc[i][j][r];
        } else {
          dst[out_row_offset(g, row, dpitch)] = from_f32<T>(apply_epilogue(acc[i][j][r] + bv, ep));
        }
      }
    }
  }
  }  // MB == 32
}

// Everything one convolution's workgroups need, as plain data (a kernel argument).
struct IgemmProblem {
  ConvGeom g;
  const void* x;
  const void* w;
  const float* bias;
  void* y;
  void* y2;  // second destination for channels [o1, o), or nullptr
  int o1;    // channels that go to y (== g.o without a second destination)
  Epilogue ep;
  int tiles_n, tiles;
  float* partial;
  int slabs_per_split, splits;
  int variant;  // mixed-group kernel only: 2 * (tile is 128x32) + (pointwise); 4..7: wave-split 32 / 16; 8, 9: 128x16 tile
};

template <typename T, int BM, int BN, int WM, int WN, int ROWB, bool PW>
__global__ __launch_bounds__(256) void conv_igemm_kernel(IgemmProblem p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[igemm_lds_bytes<BM, BN, ROWB>()];
  igemm_tile<T, BM, BN, WM, WN, ROWB, PW>(lds, p.g, static_cast<const T*>(p.x),
                                          static_cast<const T*>(p.w), p.bias,
                                          static_cast<T*>(p.y), static_cast<T*>(p.y2), p.o1, p.ep,
                                          p.tiles_n, p.tiles, p.partial, p.slabs_per_split, p.splits,
                                          (int)blockIdx.x);
}

// The fp16 128x256 tile: 128 accumulator registers per lane, so the remaining registers
// are capped to keep two waves per SIMD (one workgroup's barrier and LDS waits are then
// covered by the other's MFMAs).
template <bool PW>
__global__ __launch_bounds__(256, 2) void conv_igemm_wide_f16_kernel(IgemmProblem p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[igemm_lds_bytes<128, 256, 64>()];
  igemm_tile<__half, 128, 256, 2, 2, 64, PW>(lds, p.g, static_cast<const __half*>(p.x),
                                             static_cast<const __half*>(p.w), p.bias,
                                             static_cast<__half*>(p.y), static_cast<__half*>(p.y2), p.o1,
                                             p.ep, p.tiles_n, p.tiles, p.partial, p.slabs_per_split,
                                             p.splits, (int)blockIdx.x);
}

// Several independent convolutions in one grid: blocks [first[i], first[i+1]) work
// on problem i.  Small problems (the SSD heads) then run side by side instead of
// one launch after another, each too small to fill the chip.
constexpr int kMaxGroup = 16;
struct IgemmGroup {
  int count;
  int first[kMaxGroup + 1];
  IgemmProblem p[kMaxGroup];
};

template <typename T, int BM, int BN, int WM, int WN, int ROWB, bool PW>
__global__ __launch_bounds__(256) void conv_igemm_group_kernel(IgemmGroup grp) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[igemm_lds_bytes<BM, BN, ROWB>()];
  int i = 0;
  while (i + 1 < grp.count && (int)blockIdx.x >= grp.first[i + 1]) ++i;
  const IgemmProblem& p = grp.p[i];
  igemm_tile<T, BM, BN, WM, WN, ROWB, PW>(lds, p.g, static_cast<const T*>(p.x),
                                          static_cast<const T*>(p.w), p.bias,
                                          static_cast<T*>(p.y), static_cast<T*>(p.y2), p.o1, p.ep,
                                          p.tiles_n, p.tiles, p.partial, p.slabs_per_split, p.splits,
                                          (int)blockIdx.x - grp.first[i]);
}

template <typename T, bool PW, int TS, int U>
__device__ __forceinline__ void igemm_wave_tile(
    float* __restrict__ red, const ConvGeom& g, const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ bias, T* __restrict__ y, T* __restrict__ y2, int o1, const Epilogue& ep,
    int tiles_n, int bid);

// A group whose members differ in tile shape (64x64 or 128x32) or in being
// pointwise: each workgroup takes the code path of its own problem.  The branch is
// uniform over the workgroup; all four paths keep 16 accumulator registers per
// lane, so the register budget is that of the largest one.
template <typename T, int ROWB>
__global__ __launch_bounds__(256) void conv_igemm_mixed_kernel(IgemmGroup grp) {
  constexpr int kLds = igemm_lds_bytes<128, 32, ROWB>();  // the largest of the tiles below
  static_assert(kLds >= igemm_lds_bytes<128, 16, ROWB>() && kLds >= igemm_lds_bytes<64, 64, ROWB>(), "LDS size");
  __shared__ __attribute__((aligned(16))) unsigned char lds[kLds];
  int i = 0;
  while (i + 1 < grp.count && (int)blockIdx.x >= grp.first[i + 1]) ++i;
  const IgemmProblem& p = grp.p[i];
  const int bid = (int)blockIdx.x - grp.first[i];
#define OGLE_MIXED_CASE(V, BM, BN, WM, WN, PW)                                                  \
  case V:                                                                                       \
    igemm_tile<T, BM, BN, WM, WN, ROWB, PW>(lds, p.g, static_cast<const T*>(p.x),               \
                                            static_cast<const T*>(p.w), p.bias,                 \
                                            static_cast<T*>(p.y), static_cast<T*>(p.y2), p.o1,  \
                                            p.ep, p.tiles_n, p.tiles,                           \
                                            p.partial, p.slabs_per_split, p.splits, bid);       \
    break;
  switch (p.variant) {
    OGLE_MIXED_CASE(0, 64, 64, 2, 2, false)
    OGLE_MIXED_CASE(1, 64, 64, 2, 2, true)
    OGLE_MIXED_CASE(2, 128, 32, 4, 1, false)
    OGLE_MIXED_CASE(3, 128, 32, 4, 1, true)
    OGLE_MIXED_CASE(8, 128, 16, 4, 1, false)
    OGLE_MIXED_CASE(9, 128, 16, 4, 1, true)
#define OGLE_MIXED_WAVE(V, PW, TS)                                                               \
  case V:                                                                                       \
    /* two steps in flight only: the group kernel's register budget is the 64x64 tile's */      \
    igemm_wave_tile<T, PW, TS, 2>(reinterpret_cast<float*>(lds), p.g, static_cast<const T*>(p.x), \
                               static_cast<const T*>(p.w), p.bias, static_cast<T*>(p.y),         \
                               static_cast<T*>(p.y2), p.o1, p.ep, p.tiles_n, bid);               \
    break;
    OGLE_MIXED_WAVE(4, false, 32)
    OGLE_MIXED_WAVE(5, true, 32)
    OGLE_MIXED_WAVE(6, false, 16)
    default:
      OGLE_MIXED_WAVE(7, true, 16)
#undef OGLE_MIXED_WAVE
  }
#undef OGLE_MIXED_CASE
}

// ---------------------------------------------------------------------------
// Small problems: few output tiles, long contraction (the 1x1 ... 19x19 feature
// maps at batch 1, the extras chain, the SSD heads).  Splitting K across workgroups
// needs a second launch to add the parts, and a dependent launch costs more than
// these convolutions themselves.  Here the split stays inside the workgroup: a
// workgroup owns one 32x32 (or 16x16) output tile, its four waves each contract a quarter of K,
// and the four partial tiles are added through LDS in wave order (a fixed order, so
// the result does not depend on timing).  A wave feeds its MFMAs straight from
// global memory: both operands are K-contiguous, so the 16 bytes a lane loads are
// exactly its share of an MFMA operand (fp32: four k of an 8-wide group, fp16: eight
// k of a 16-wide one); no LDS and no barrier in the K loop, and one wave per SIMD
// can keep its MFMA pipe busy because consecutive MFMAs into one accumulator issue
// back to back.  Operands are re-read by every tile that shares them, which the L2
// absorbs at these sizes.
constexpr int kWaveRedBytes = 4 * 32 * 36 * 4;  // four staged 32x32 partial tiles, padded rows

// U: steps of loads in flight per register set (two sets).
template <typename T, bool PW, int TS, int U>
__device__ __forceinline__ void igemm_wave_tile(
    float* __restrict__ red, const ConvGeom& g, const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ bias, T* __restrict__ y, T* __restrict__ y2, int o1, const Epilogue& ep,
    int tiles_n, int bid) {
  typedef WaveMma<T, TS> M;
  constexpr int ESZ = (int)sizeof(T);
  constexpr int VE = 16 / ESZ;          // elements per 16-byte load
  constexpr int QN = 64 / TS;           // lane groups along k
  constexpr int KSTEP = QN * VE;        // k covered by one step
  constexpr int PITCH = TS + 4;         // floats per row of a staged partial tile
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  // MFMA operand order: lane = q * TS + row.  Loads use the other order, lane =
  // row * QN + q, so that the QN lanes of a row read one contiguous run (the vector
  // cache takes one access per contiguous run, and one per lane otherwise, which is
  // what bounds these problems); a lane permute puts the data into MFMA order.  The
  // 16x16 form of a non-pointwise problem is only chosen for tiny maps that wait on
  // latency, not on the cache, and the permutes only lengthen their chain: those load
  // in MFMA order.
  const int mt = lane % TS, mq = lane / TS;        // MFMA order (also the result layout)
  constexpr bool PERM = PW || TS == 32;
  const int lt = PERM ? lane / QN : mt, lq = PERM ? lane % QN : mq;        // load order
  const int permute_from = (mt * QN + mq) * 4;     // byte address for ds_bpermute
  const int tile_n = bid % tiles_n, tile_m = bid / tiles_n;
  const int m = tile_m * TS + lt;       // the A row this lane loads
  const int col = tile_n * TS + lt;     // the B row (output channel) this lane loads
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x, g.x_bytes);
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(w, g.w_bytes);

  const int csteps = (g.c + KSTEP - 1) / KSTEP;   // steps per tap
  const int steps = g.k * g.k * csteps;
  const int s_begin = (int)(((long)steps * wave) / 4), s_end = (int)(((long)steps * (wave + 1)) / 4);

  // row geometry of this lane
  int iy0 = 0, ix0 = 0;
  unsigned img = 0;
  const bool row_ok = m < g.m_total;
  if (PW) {
    img = (unsigned)m * (unsigned)(g.c * ESZ);
  } else {
    const int ox = m % g.ow;
    const int t = m / g.ow;
    const int oy = t % g.oh;
    const int b = t / g.oh;
    img = (unsigned)b * (unsigned)(g.h * g.w * g.c * ESZ);
    iy0 = oy * g.stride - g.pad;
    ix0 = ox * g.stride - g.pad;
  }
  const unsigned wrow = (unsigned)col * (unsigned)(g.k * g.k * g.c * ESZ);
  const bool col_ok = col < g.o;

  // load cursor: (tap, channel step) of the next step to request
  int l_tap = s_begin / csteps, l_cs = s_begin - l_tap * csteps;
  unsigned a_tap = kOutOfRange, b_tap = kOutOfRange;
  auto enter_tap = [&](int tap) {
    if (PW) {
      a_tap = row_ok ? img : kOutOfRange;
    } else {
      const int ky = tap / g.k, kx = tap - ky * g.k;
      const int iy = iy0 + ky * g.dil, ix = ix0 + kx * g.dil;
      const bool in = row_ok && iy >= 0 && iy < g.h && ix >= 0 && ix < g.w;
      a_tap = in ? img + (unsigned)((iy * g.w + ix) * g.c * ESZ) : kOutOfRange;
    }
    b_tap = col_ok ? wrow + (unsigned)(tap * g.c * ESZ) : kOutOfRange;
  };
  enter_tap(l_tap);

  u32x4 ra[2][U], rb[2][U];
  int requested = s_begin;
#define OGLE_WAVE_LOAD(SET)                                                                      \
  _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                \
    const int cel = l_cs * KSTEP + lq * VE;                                                      \
    const bool ok = requested < s_end && cel < g.c;                                              \
    const unsigned ao = ok && a_tap != kOutOfRange ? a_tap + (unsigned)(cel * ESZ) : kOutOfRange; \
    const unsigned bo = ok && b_tap != kOutOfRange ? b_tap + (unsigned)(cel * ESZ) : kOutOfRange; \
    ra[SET][u] = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)ao, 0, 0);                       \
    rb[SET][u] = __builtin_amdgcn_raw_buffer_load_b128(rw, (int)bo, 0, 0);                       \
    ++requested;                                                                                 \
    if (++l_cs == csteps) {                                                                      \
      l_cs = 0;                                                                                  \
      ++l_tap;                                                                                   \
      enter_tap(l_tap);                                                                          \
    }                                                                                            \
  }
#define OGLE_WAVE_MMA(SET)                                                                       \
  _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                \
    u32x4 av, bv;                                                                                \
    _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                              \
      av[e] = PERM ? (unsigned)__builtin_amdgcn_ds_bpermute(permute_from, (int)ra[SET][u][e]) : ra[SET][u][e]; \
      bv[e] = PERM ? (unsigned)__builtin_amdgcn_ds_bpermute(permute_from, (int)rb[SET][u][e]) : rb[SET][u][e]; \
    }                                                                                            \
    M::run(av, bv, acc);                                                                         \
  }

  typename M::Acc acc;
#pragma unroll
  for (int r = 0; r < M::REGS; ++r) acc[r] = 0.f;

  // chunks of U steps, two register sets: the next chunk is in flight while the
  // current one is multiplied; steps past s_end load zeros
  // (the scheduling barriers keep a whole chunk of loads ahead of the MFMAs that
  // consume the previous one; left alone the compiler sinks the loads next to their
  // uses and the wave then waits for memory once per step)
  OGLE_WAVE_LOAD(0);
  for (int s = s_begin; s < s_end; s += 2 * U) {
    OGLE_WAVE_LOAD(1);
    __builtin_amdgcn_sched_barrier(0);
    OGLE_WAVE_MMA(0);
    __builtin_amdgcn_sched_barrier(0);
    OGLE_WAVE_LOAD(0);
    __builtin_amdgcn_sched_barrier(0);
    OGLE_WAVE_MMA(1);
    __builtin_amdgcn_sched_barrier(0);
  }
#undef OGLE_WAVE_LOAD
#undef OGLE_WAVE_MMA

  // the four partial tiles, then their sum in wave order.  Result layout: register r
  // of lane l is row 8*(r/4) + 4*(l/32) + r%4 (32x32) or 4*(l/16) + r (16x16), column l % TS.
  float* mine = red + wave * (TS * PITCH);
#pragma unroll
  for (int r = 0; r < M::REGS; ++r) {
    const int row = TS == 32 ? (r >> 2) * 8 + mq * 4 + (r & 3) : mq * 4 + r;
    mine[row * PITCH + mt] = acc[r];
  }
  __syncthreads();
  constexpr int VPR = TS / 4;             // 4-element groups per row
  if (tid >= TS * VPR) return;            // TS 16: 64 threads finish the tile
  const int orow = tid / VPR, ocol = (tid % VPR) * 4;
  const float* p0 = red + orow * PITCH + ocol;
  float4 sum = *reinterpret_cast<const float4*>(p0);
#pragma unroll
  for (int wv = 1; wv < 4; ++wv) {
    const float4 t = *reinterpret_cast<const float4*>(p0 + wv * (TS * PITCH));
    sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w;
  }
  const int grow = tile_m * TS + orow;
  const int gcol = tile_n * TS + ocol;
  if (grow >= g.m_total || gcol >= g.o) return;
  float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (gcol + q < g.o) v[q] = apply_epilogue(v[q] + (bias != nullptr ? bias[gcol + q] : 0.f), ep);
  }
  if (y2 != nullptr) {
    // two destinations: element by element, each channel to its own tensor
    const int o2 = g.o - o1;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int c = gcol + q;
      if (c >= g.o) continue;
      if (c < o1) y[(long)grow * o1 + c] = from_f32<T>(v[q]);
      else y2[(long)grow * o2 + (c - o1)] = from_f32<T>(v[q]);
    }
    return;
  }
  T* dst = y + out_row_offset(g, grow, g.o) + gcol;
  if ((g.o & 3) == 0 && (g.oimg & 3) == 0) {
    if constexpr (sizeof(T) == 4) {
      store_result16(dst, make_float4(v[0], v[1], v[2], v[3]));
    } else {
      const __half2 lo = __floats2half2_rn(v[0], v[1]), hi = __floats2half2_rn(v[2], v[3]);
      uint2 packed;
      packed.x = *reinterpret_cast<const unsigned*>(&lo);
      packed.y = *reinterpret_cast<const unsigned*>(&hi);
      store_result8(dst, packed);
    }
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (gcol + q < g.o) dst[q] = from_f32<T>(v[q]);
  }
}

template <typename T, bool PW, int TS>
__global__ __launch_bounds__(256) void conv_igemm_wave_kernel(IgemmProblem p) {
  __shared__ __attribute__((aligned(16))) float red[kWaveRedBytes / 4];
  igemm_wave_tile<T, PW, TS, 4>(red, p.g, static_cast<const T*>(p.x), static_cast<const T*>(p.w),
                             p.bias, static_cast<T*>(p.y), static_cast<T*>(p.y2), p.o1, p.ep, p.tiles_n,
                             (int)blockIdx.x);
}

struct ReduceProblem {
  const float* partial;  // [splits][m][opitch]
  const float* bias;
  void* y;
  void* y2;   // second destination for channels [o1, o), or nullptr
  long mn;    // m * o output elements
  int o, o1, opitch, splits;
  Epilogue ep;
  int lanes;  // lanes per output element (1, 2, 4 or 8)
  long oimg;  // elements between the outputs of consecutive images in y; 0: dense
  int hw;     // output rows per image
};
struct ReduceGroup {
  int count;
  int first[kMaxGroup + 1];
  ReduceProblem p[kMaxGroup];
};

// Sums the split-K partials, then bias and activation.  A work item is four consecutive
// channels of one output row (the partial rows are padded to a multiple of four floats,
// so it is one 16-byte load per split), shared by LANES consecutive lanes: lane q adds
// splits q, q+LANES, ... in ascending order and the LANES partial sums are then combined
// in a fixed butterfly order, so the result depends on neither timing nor grid shape.
// Spreading the splits over lanes keeps many loads in flight when there are few outputs
// but many splits.
template <typename T, int LANES>
__device__ __forceinline__ void splitk_reduce_block(const ReduceProblem& r, int bid) {
  const int q = threadIdx.x % LANES;
  const int gpr = r.opitch >> 2;       // four-channel groups per row
  const long rows = r.mn / r.o;
  const long idx = (long)bid * (blockDim.x / LANES) + threadIdx.x / LANES;
  const bool live = idx < rows * gpr;  // dead lanes still take part in the shuffles
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  const long row = idx / gpr;
  const int col = (int)(idx - row * gpr) * 4;
  if (live) {
    const float* src = r.partial + row * r.opitch + col;
    const long zstride = rows * r.opitch;
#pragma unroll 4
    for (int z = q; z < r.splits; z += LANES) {
      const float4 t = *reinterpret_cast<const float4*>(src + (long)z * zstride);
      acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
    }
  }
#pragma unroll
  for (int d = 1; d < LANES; d <<= 1) {
    acc.x += __shfl_xor(acc.x, d, 64);
    acc.y += __shfl_xor(acc.y, d, 64);
    acc.z += __shfl_xor(acc.z, d, 64);
    acc.w += __shfl_xor(acc.w, d, 64);
  }
  if (!live || q != 0) return;
  float v[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (col + e < r.o) v[e] = apply_epilogue(v[e] + (r.bias != nullptr ? r.bias[col + e] : 0.f), r.ep);
  // where this row's channels start in y
  long at = row * r.o1;
  if (r.oimg != 0) {
    const long b = row / r.hw;
    at = b * r.oimg + (row - b * r.hw) * r.o;
  }
  if (sizeof(T) == 4 && r.y2 == nullptr && (r.o & 3) == 0 && (r.oimg & 3) == 0) {
    store_result16(static_cast<float*>(r.y) + at + col, make_float4(v[0], v[1], v[2], v[3]));
    return;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int c = col + e;
    if (c >= r.o) continue;
    if (c < r.o1) static_cast<T*>(r.y)[at + c] = from_f32<T>(v[e]);
    else static_cast<T*>(r.y2)[row * (r.o - r.o1) + (c - r.o1)] = from_f32<T>(v[e]);
  }
}

template <typename T, int LANES>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(ReduceProblem r) {
  splitk_reduce_block<T, LANES>(r, (int)blockIdx.x);
}

// The reductions of a whole group in one grid; each workgroup uses the lane count
// its own problem was planned with.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_group_kernel(ReduceGroup grp) {
  int i = 0;
  while (i + 1 < grp.count && (int)blockIdx.x >= grp.first[i + 1]) ++i;
  const ReduceProblem& r = grp.p[i];
  const int bid = (int)blockIdx.x - grp.first[i];
  switch (r.lanes) {
    case 8: splitk_reduce_block<T, 8>(r, bid); break;
    case 4: splitk_reduce_block<T, 4>(r, bid); break;
    case 2: splitk_reduce_block<T, 2>(r, bid); break;
    default: splitk_reduce_block<T, 1>(r, bid); break;
  }
}

// Tile configurations (BM, BN, waves along M, waves along N).
enum TileCfg {
  CFG_128x128 = 0, CFG_128x64 = 1, CFG_64x64 = 2, CFG_128x32 = 3, CFG_WAVE32 = 4, CFG_WAVE16 = 5,
  CFG_128x96 = 6, CFG_128x160 = 7,  // all output channels of a narrow, long-K problem in one tile
  CFG_128x256 = 8,                   // fp16 storage: 64x128 per wave, 64-byte K slabs
  CFG_128x16 = 9                     // at most 16 output channels: 16x16 MFMA blocks
};
constexpr int kCfgBM[] = {128, 128, 64, 128, 32, 16, 128, 128, 128, 128};
constexpr int kCfgBN[] = {128, 64, 64, 32, 32, 16, 96, 160, 256, 16};
constexpr int kRowBytesF16Wide = 64;  // K bytes per tile row per slab of CFG_128x256

struct IgemmPlan {
  int cfg;
  int splits;
  bool rows_on_xcd;  // split-K work layout: tile rows, not K ranges, pinned to an XCD
  int slabs_per_split;
  int ktiles;
  int cchunks;
  size_t workspace_bytes;  // splits * M * N floats when splits > 1
};

constexpr long kComputeUnits = 256;
constexpr int kRowBytesF32 = 64;   // bytes of K per tile row per slab, fp32

bool is_pointwise(const OgleConvArgs& a);
bool is_wave(int cfg);

// Picks the output tile and the K split.  Problems with few output
// tiles but a long contraction (the SSD heads, the small feature maps) are split
// along K until the grid fills the chip, provided a workspace was supplied.
IgemmPlan plan_igemm(const OgleConvArgs& a, long m, bool allow_split) {
  IgemmPlan p{};
  const int esz = a.dtype == OGLE_F16 ? 2 : 4;
  const int rowb = a.dtype == OGLE_F16 ? 128 : kRowBytesF32;
  const int epr = rowb / esz;
  p.cchunks = (a.in_c + epr - 1) / epr;
  p.ktiles = a.kernel_size * a.kernel_size * p.cchunks;
  auto tiles = [&](int cfg) {
    return ((m + kCfgBM[cfg] - 1) / kCfgBM[cfg]) * ((a.out_c + kCfgBN[cfg] - 1) / kCfgBN[cfg]);
  };
  // Measured on MI355X: 64x64 tiles (eight waves per SIMD resident) match or beat
  // the larger tiles on every layer of the network because they quantise better
  // over 256 CUs and hide latency with occupancy; 128x128 only pays off once there
  // are enough tiles for several rounds.
  // fp16 storage: an MFMA does sixteen times the work per operand byte, so the
  // 64x64 tile is bound by LDS traffic and instruction issue; 128x128 pays off as soon
  // as its tiles cover the compute units.
  const long big_tiles_wanted = a.dtype == OGLE_F16 ? kComputeUnits : 4 * kComputeUnits;
  // Narrow outputs with a long contraction (the SSD heads, box and class head of a feature
  // map fused: 75 or 150 channels, K = 2304 ... 9216): one tile column holds every output
  // channel, so the input is gathered once instead of once per 64-channel tile column, and
  // 96 / 160 columns waste far less of the MFMA work than two or three 64-wide tiles.
  const bool narrow_long = a.dtype == OGLE_F32 && p.ktiles >= 32 &&
                           ((a.out_c > 64 && a.out_c <= 96) || (a.out_c > 128 && a.out_c <= 160));
  if (narrow_long) {
    p.cfg = a.out_c <= 96 ? CFG_128x96 : CFG_128x160;
  } else if (a.dtype == OGLE_F16 && a.out_c >= 256 && tiles(CFG_128x256) >= 2 * kComputeUnits) {
    // fp16 storage: one MFMA does sixteen times the work per operand byte, and a wave that
    // owns 64x64 outputs reads its operands from LDS as fast as the MFMA pipe consumes them.
    // A wave with 64x128 outputs reads a third less per MFMA and the tile pulls a quarter
    // less from L2; 64-byte slabs keep two such workgroups per compute unit.  Measured on
    // MI355X: M = 46208, K = N = 1024 gains 8 % (610 -> 662 TFLOP/s), but with fewer than two
    // tiles per compute unit (M = 11552, N = 1024: 364 tiles) the second round is mostly
    // empty and the 128x128 tile stays ahead (480 against 448 TFLOP/s).
    p.cfg = CFG_128x256;
    const int epr2 = kRowBytesF16Wide / esz;
    p.cchunks = (a.in_c + epr2 - 1) / epr2;
    p.ktiles = a.kernel_size * a.kernel_size * p.cchunks;
  } else if (a.out_c <= 16) {
    p.cfg = CFG_128x16;
  } else if (a.out_c <= 32) {
    p.cfg = CFG_128x32;
  } else if (a.out_c > 64 && tiles(CFG_128x128) >= big_tiles_wanted) {
    p.cfg = CFG_128x128;
  } else {
    p.cfg = CFG_64x64;
  }
  p.splits = 1;
  const long t = tiles(p.cfg);
  long sp = 1;
  bool exact_split = false;  // sp was chosen by the search below: any count is fine
  if (allow_split && narrow_long && t < 2 * kComputeUnits) {
    // One tile column, few tile rows, a long K: the K split decides how evenly the chip is
    // filled.  Workgroups are (tile, K range) pairs dealt to 256 compute units, each doing
    // ceil(ktiles / s) slabs plus a fixed cost (first loads, epilogue: about `fixed` slabs);
    // take the s with the shortest estimated time, partial-sum traffic as the tie break.
    const double fixed = p.cfg == CFG_128x96 ? 6.0 : 4.0;
    double best = 1e30;
    for (long s = 1; s <= 64 && p.ktiles / s >= 8; ++s) {
      const long rounds = (t * s + kComputeUnits - 1) / kComputeUnits;
      const double cost = (double)rounds * ((double)((p.ktiles + s - 1) / s) + fixed) + 0.25 * (double)s;
      if (cost < best - 1e-9) {
        best = cost;
        sp = s;
      }
    }
    exact_split = true;
  } else if (allow_split && 2 * t <= kComputeUnits && p.ktiles >= 8) {
    // too few tiles to occupy every compute unit: about three workgroups per unit,
    // at least four slabs per split
    const long want = (3 * kComputeUnits + t - 1) / t;
    const long most = p.ktiles / 4;
    sp = want < most ? want : most;
  } else if (allow_split && t < 8 * kComputeUnits && p.ktiles >= 128) {
    // a few long workgroups per unit quantise badly (one unit gets two, its
    // neighbour one) and leave one wave per SIMD: cut the long contraction so that
    // about eight shorter workgroups land on every unit, 32 slabs or more each
    const long want = (8 * kComputeUnits + t - 1) / t;
    const long most = p.ktiles / 32;
    sp = want < most ? want : most;
  }
  if (sp > 64) sp = 64;
  // the kernel's XCD-aware work layout wants a divisor or a multiple of 8
  if (exact_split) {}
  else if (sp >= 8) sp -= sp % 8;
  else if (sp >= 4) sp = 4;
  else if (sp >= 2) sp = 2;
  if (sp >= 2) p.splits = (int)sp;
  // A small contraction that would be split across workgroups goes to the wave-split
  // kernel instead (the split stays inside the workgroup: no workspace, no second
  // launch), whether or not a workspace was offered.  Measured on MI355X against
  // split-K + reduce: the 32x32 form wins once its tiles cover half the chip, for
  // K <= 1024 pointwise and K <= 512 otherwise; the 16x16 form wins for pointwise
  // K <= 1024 while its tiles stay under two per compute unit, and for K <= 1536 while they
  // stay under one per unit (3x3x256 <- 5x5x128 at batch 16: 7.0 against 9.5 us); a longer K
  // per wave is a serial chain of MFMAs and loses to the split across workgroups.
  {
    const long k_total = (long)a.kernel_size * a.kernel_size * a.in_c;
    const bool pw = is_pointwise(a);
    const bool would_split = (2 * t <= kComputeUnits && p.ktiles >= 8) ||
                             (t < 8 * kComputeUnits && p.ktiles >= 128);
    const long t32 = tiles(CFG_WAVE32), t16 = tiles(CFG_WAVE16);
    const bool small16 = (pw && k_total <= 1024 && t16 <= 2 * kComputeUnits) ||
                         (k_total <= 1536 && t16 <= kComputeUnits);
    // other than pointwise: K <= 512, or up to 2304 while every 32x32 tile has a compute unit
    // to itself (5x5x512 <- 10x10x256, 3x3 stride 2, at batch 16: 19.8 against 21.6 us)
    const long k32cap = t32 <= kComputeUnits ? 2304 : 512;
    if (narrow_long) {
      // stays on the wide tile
    } else if (would_split && !small16 && k_total <= (pw ? 1024 : k32cap) && t32 >= kComputeUnits / 2 &&
        t32 <= 4 * kComputeUnits) {
      p.cfg = CFG_WAVE32;
      p.splits = 1;
    } else if (would_split && small16) {
      p.cfg = CFG_WAVE16;
      p.splits = 1;
    }
  }
  p.slabs_per_split = (p.ktiles + p.splits - 1) / p.splits;
  if (p.splits > 1) {
    p.slabs_per_split += p.slabs_per_split & 1;  // the K loop runs slab pairs
    p.splits = (p.ktiles + p.slabs_per_split - 1) / p.slabs_per_split;  // no empty ranges
  }
  // (a split past the end of K would only add zeros; rounding splits down keeps the
  // divisor-or-multiple-of-8 shape, so empty splits are simply avoided by the cap above)
  // partial sums are kept in rows of the channel count rounded up to four
  p.workspace_bytes =
      p.splits > 1 ? (size_t)p.splits * (size_t)m * ((a.out_c + 3) & ~3) * sizeof(float) : 0;
  // Which operand an XCD's L2 should keep to itself: with K ranges pinned to XCDs the input is
  // fetched by all eight L2s and the filter by one, with tile rows pinned it is the other way
  // round (the rocprofv3 FETCH_SIZE of the 19x19x512 class head fell from 8.5x its input to
  // about the input plus eight filters).
  {
    const long x_bytes = (long)a.n * a.in_h * a.in_w * a.in_c * esz;
    const long w_bytes = (long)a.out_c * a.kernel_size * a.kernel_size * a.in_c * esz;
    // whole tile rows per XCD: only when they spread evenly (within a tenth) over the eight
    const long tiles_m = (m + kCfgBM[p.cfg] - 1) / kCfgBM[p.cfg];
    const bool even = ((tiles_m + 7) / 8) * 8 * 10 <= tiles_m * 11;
    p.rows_on_xcd = p.splits > 1 && !is_wave(p.cfg) && x_bytes > w_bytes && even;
  }
  return p;
}

bool is_wave(int cfg) { return cfg == CFG_WAVE32 || cfg == CFG_WAVE16; }
int tile_bm(int cfg) { return kCfgBM[cfg]; }
int tile_bn(int cfg) { return kCfgBN[cfg]; }

// Grid size of one problem under the kernel's XCD-aware work layout.
unsigned grid_blocks(const IgemmPlan& p, int tiles_m, int tiles_n) {
  const int tiles = tiles_m * tiles_n;
  if (p.splits == 1) return 8u * (unsigned)((tiles_m + 7) / 8) * (unsigned)tiles_n;
  if (p.rows_on_xcd) return 8u * (unsigned)((tiles_m + 7) / 8) * (unsigned)tiles_n * (unsigned)p.splits;
  if (p.splits != 2 && p.splits != 4) return (unsigned)tiles * (unsigned)p.splits;
  const int xpz = 8 / p.splits;
  return 8u * (unsigned)((tiles + xpz - 1) / xpz);
}

bool igemm_eligible(const OgleConvArgs& a, long* m_out) {
  if (a.group != 1) return false;
  const int ve = a.dtype == OGLE_F16 ? 8 : 4;
  if (a.in_c % ve != 0) return false;
  if ((long)a.kernel_size * a.kernel_size * a.in_c < 32) return false;
  const long m = (long)a.n * a.out_h * a.out_w;
  if (m <= 0 || m > 0x7fffffffL) return false;
  // operands are addressed with 32-bit byte offsets through buffer loads
  const long esz = a.dtype == OGLE_F16 ? 2 : 4;
  const long lim = 0x7fffffffL;
  if ((long)a.n * a.in_h * a.in_w * a.in_c * esz > lim) return false;
  if ((long)a.out_c * a.kernel_size * a.kernel_size * a.in_c * esz > lim) return false;
  *m_out = m;
  return true;
}

bool is_pointwise(const OgleConvArgs& a) {
  return a.kernel_size == 1 && a.stride == 1 && a.padding == 0;
}

// The plan the launch will use: split-K only with a workspace that is large enough.
IgemmPlan final_plan(const OgleConvArgs& a, long m) {
  IgemmPlan p = plan_igemm(a, m, a.workspace_dev != nullptr);
  if (p.workspace_bytes > a.workspace_bytes) p = plan_igemm(a, m, false);
  return p;
}

struct Prepared {
  IgemmProblem prob;
  ReduceProblem red;
  unsigned grid;
  unsigned reduce_grid;
  int reduce_lanes;
};

Prepared prepare(const OgleConvArgs& a, long m, const IgemmPlan& p) {
  Prepared out{};
  ConvGeom& g = out.prob.g;
  g.n = a.n; g.h = a.in_h; g.w = a.in_w; g.c = a.in_c;
  g.oh = a.out_h; g.ow = a.out_w; g.o = a.out_c;
  g.k = a.kernel_size; g.stride = a.stride; g.pad = a.padding; g.dil = a.dilation;
  g.m_total = (int)m;
  g.cchunks = p.cchunks;
  g.ktiles = p.ktiles;
  const long esz = a.dtype == OGLE_F16 ? 2 : 4;
  g.x_bytes = (unsigned)((long)a.n * a.in_h * a.in_w * a.in_c * esz);
  g.w_bytes = (unsigned)((long)a.out_c * a.kernel_size * a.kernel_size * a.in_c * esz);
  g.oimg = a.out_image_stride == (long)a.out_h * a.out_w * a.out_c ? 0 : a.out_image_stride;
  const int tiles_m = (g.m_total + tile_bm(p.cfg) - 1) / tile_bm(p.cfg);
  const int tiles_n = (g.o + tile_bn(p.cfg) - 1) / tile_bn(p.cfg);
  out.prob.x = a.input_dev;
  out.prob.w = a.filter_dev;
  out.prob.bias = a.bias_dev;
  out.prob.y = a.output_dev;
  out.prob.y2 = a.output2_dev;
  out.prob.o1 = a.output2_dev != nullptr ? a.out_c_split : a.out_c;
  out.prob.ep = make_epilogue(a.act, a.min_value, a.max_value, a.act_variant);
  out.prob.tiles_n = tiles_n;
  out.prob.tiles = tiles_m * tiles_n;
  out.prob.partial = p.splits > 1 ? static_cast<float*>(a.workspace_dev) : nullptr;
  out.prob.slabs_per_split = p.slabs_per_split;
  out.prob.splits = p.rows_on_xcd ? -p.splits : p.splits;
  out.prob.variant = (p.cfg == CFG_WAVE32 ? 4 : p.cfg == CFG_WAVE16 ? 6 : p.cfg == CFG_128x32 ? 2 :
                      p.cfg == CFG_128x16 ? 8 : 0) +
                     (is_pointwise(a) ? 1 : 0);
  if (is_wave(p.cfg)) {
    out.grid = (unsigned)(tiles_m * tiles_n);
    return out;
  }
  out.grid = grid_blocks(p, tiles_m, tiles_n);
  if (p.splits > 1) {
    const long mn = (long)g.m_total * g.o;
    // enough lanes per output that the grid still has about a thousand waves
    const long items = (long)g.m_total * (((g.o + 3) & ~3) / 4);  // four channels each
    int lanes = 1;
    while (lanes < 8 && lanes * 2 <= p.splits && items * lanes < 64L * 1024) lanes *= 2;
    out.red = ReduceProblem{out.prob.partial, a.bias_dev, a.output_dev, a.output2_dev, mn, g.o,
                            out.prob.o1, (g.o + 3) & ~3, p.splits, out.prob.ep, lanes, g.oimg,
                            g.oh * g.ow};
    out.reduce_lanes = lanes;
    out.reduce_grid = (unsigned)((items * lanes + 255) / 256);
  }
  return out;
}

// Instantiates kernel `K<T, BM, BN, WM, WN, ROWB, PW>` for a runtime (dtype, cfg, pw).
#define OGLE_IGEMM_DISPATCH(K, dtype, cfg, pw, ...)                                          \
  do {                                                                                       \
    if ((dtype) == OGLE_F16) {                                                               \
      OGLE_IGEMM_DISPATCH_T(K, __half, 128, cfg, pw, __VA_ARGS__);                           \
    } else {                                                                                 \
      OGLE_IGEMM_DISPATCH_T(K, float, kRowBytesF32, cfg, pw, __VA_ARGS__);                   \
    }                                                                                        \
  } while (0)
#define OGLE_IGEMM_DISPATCH_T(K, T, ROWB, cfg, pw, ...)                                      \
  do {                                                                                       \
    if (pw) {                                                                                \
      OGLE_IGEMM_DISPATCH_C(K, T, ROWB, true, cfg, __VA_ARGS__);                             \
    } else {                                                                                 \
      OGLE_IGEMM_DISPATCH_C(K, T, ROWB, false, cfg, __VA_ARGS__);                            \
    }                                                                                        \
  } while (0)
#define OGLE_IGEMM_DISPATCH_C(K, T, ROWB, PW, cfg, grid, s, arg)                             \
  switch (cfg) {                                                                             \
    case CFG_128x128:                                                                        \
      launch((K<T, 128, 128, 2, 2, ROWB, PW>), dim3(grid), dim3(256), 0, s, arg); \
      break;                                                                                 \
    case CFG_128x64:                                                                         \
      launch((K<T, 128, 64, 2, 2, ROWB, PW>), dim3(grid), dim3(256), 0, s, arg);  \
      break;                                                                                 \
    case CFG_64x64:                                                                          \
      launch((K<T, 64, 64, 2, 2, ROWB, PW>), dim3(grid), dim3(256), 0, s, arg);   \
      break;                                                                                 \
    case CFG_128x96:                                                                         \
      launch((K<T, 128, 96, 4, 1, ROWB, PW>), dim3(grid), dim3(256), 0, s, arg);  \
      break;                                                                                 \
    case CFG_128x160:                                                                        \
      launch((K<T, 128, 160, 4, 1, ROWB, PW>), dim3(grid), dim3(256), 0, s, arg); \
      break;                                                                                 \
    case CFG_128x16:                                                                         \
      launch((K<T, 128, 16, 4, 1, ROWB, PW>), dim3(grid), dim3(256), 0, s, arg);  \
      break;                                                                                 \
    default:                                                                                 \
      launch((K<T, 128, 32, 4, 1, ROWB, PW>), dim3(grid), dim3(256), 0, s, arg);  \
      break;                                                                                 \
  }

// One problem, one grid of the LDS-tiled kernel.
void launch_single(int dtype, int cfg, bool pw, unsigned grid, hipStream_t s, const IgemmProblem& prob) {
  if (cfg == CFG_128x256) {  // fp16 storage only (plan_igemm)
    if (pw) launch(conv_igemm_wide_f16_kernel<true>, dim3(grid), dim3(256), 0, s, prob);
    else launch(conv_igemm_wide_f16_kernel<false>, dim3(grid), dim3(256), 0, s, prob);
    return;
  }
  OGLE_IGEMM_DISPATCH(conv_igemm_kernel, dtype, cfg, pw, grid, s, prob);
}

void launch_wave(int dtype, bool pw, int cfg, const Prepared& pr, hipStream_t s) {
  const dim3 grid(pr.grid), block(256);
#define OGLE_WAVE_LAUNCH(T, PW, TS) \
  launch((conv_igemm_wave_kernel<T, PW, TS>), grid, block, 0, s, pr.prob)
#define OGLE_WAVE_PICK(T)                                                 \
  if (cfg == CFG_WAVE32) {                                                \
    if (pw) OGLE_WAVE_LAUNCH(T, true, 32); else OGLE_WAVE_LAUNCH(T, false, 32); \
  } else {                                                                \
    if (pw) OGLE_WAVE_LAUNCH(T, true, 16); else OGLE_WAVE_LAUNCH(T, false, 16); \
  }
  if (dtype == OGLE_F16) {
    OGLE_WAVE_PICK(__half)
  } else {
    OGLE_WAVE_PICK(float)
  }
#undef OGLE_WAVE_PICK
#undef OGLE_WAVE_LAUNCH
}

template <typename T>
void launch_reduce_single(const Prepared& pr, hipStream_t s) {
  const dim3 grid(pr.reduce_grid), block(256);
  switch (pr.reduce_lanes) {
    case 8: launch((splitk_reduce_kernel<T, 8>), grid, block, 0, s, pr.red); break;
    case 4: launch((splitk_reduce_kernel<T, 4>), grid, block, 0, s, pr.red); break;
    case 2: launch((splitk_reduce_kernel<T, 2>), grid, block, 0, s, pr.red); break;
    default: launch((splitk_reduce_kernel<T, 1>), grid, block, 0, s, pr.red); break;
  }
}

}  // namespace

bool conv_igemm_takes(const OgleConvArgs& a) {
  long m = 0;
  return igemm_eligible(a, &m);
}

size_t conv_igemm_workspace_bytes(const OgleConvArgs& a) {
  long m = 0;
  if (!igemm_eligible(a, &m)) return 0;
  if (f16_async_config(a) >= 0) return 0;
  return plan_igemm(a, m, true).workspace_bytes;
}

int32_t launch_conv_igemm(const OgleConvArgs& a, hipStream_t s) {
  long m = 0;
  if (!igemm_eligible(a, &m)) return OGLE_ERR_UNSUPPORTED;
  if (f16_async_config(a) >= 0) return launch_pw_gemm_f16_async(a, s);
  const IgemmPlan p = final_plan(a, m);
  const Prepared pr = prepare(a, m, p);
  const bool pw = is_pointwise(a);
  if (is_wave(p.cfg)) {
    launch_wave(a.dtype, pw, p.cfg, pr, s);
    return check_launch("conv_igemm_wave");
  }
  launch_single(a.dtype, p.cfg, pw, pr.grid, s, pr.prob);
  int32_t st = check_launch("conv_igemm");
  if (st != OGLE_OK || p.splits == 1) return st;
  if (a.dtype == OGLE_F16) launch_reduce_single<__half>(pr, s);
  else launch_reduce_single<float>(pr, s);
  return check_launch("splitk_reduce");
}

// Launches `count` mutually independent convolutions.  Those the implicit-GEMM
// kernel takes go out as ONE grid (plus one grid for all of their split-K
// reductions) per storage type: a group whose members share the kernel
// instantiation uses that instantiation, a mixed group of 64x64 and 128x32 tiles the
// kernel that branches per workgroup; 128x128-tile problems fill the chip on their
// own and are launched singly.  The others are launched one by one through `fallback`.
int32_t launch_conv_batch(const OgleConvArgs* args, int count, hipStream_t s,
                          int32_t (*fallback)(const OgleConvArgs&, hipStream_t),
                          int32_t* reduce_pending) {
  struct Item {
    int dtype, cfg;
    bool pw;
    Prepared pr;
  };
  std::vector<Item> items;
  for (int i = 0; i < count; ++i) {
    if (reduce_pending != nullptr) reduce_pending[i] = 0;
    long m = 0;
    if (!igemm_eligible(args[i], &m)) {
      const int32_t st = fallback(args[i], s);
      if (st != OGLE_OK) return st;
      continue;
    }
    if (f16_async_config(args[i]) >= 0) {  // fills the chip on its own: its own launch
      const int32_t st = launch_pw_gemm_f16_async(args[i], s);
      if (st != OGLE_OK) return st;
      continue;
    }
    const IgemmPlan p = final_plan(args[i], m);
    items.push_back(Item{args[i].dtype, p.cfg, is_pointwise(args[i]), prepare(args[i], m, p)});
    if (reduce_pending != nullptr && p.splits > 1) reduce_pending[i] = 1;
  }
  auto mixable = [](const Item& it) {
    return it.cfg == CFG_64x64 || it.cfg == CFG_128x32 || it.cfg == CFG_128x16 || is_wave(it.cfg);
  };
  std::vector<bool> done(items.size(), false);
  for (size_t a0 = 0; a0 < items.size(); ++a0) {
    if (done[a0]) continue;
    IgemmGroup grp{};
    ReduceGroup red{};
    const Item& head = items[a0];
    bool uniform = true;
    for (size_t b0 = a0; b0 < items.size() && grp.count < kMaxGroup; ++b0) {
      const Item& it = items[b0];
      if (done[b0] || it.dtype != head.dtype) continue;
      const bool same = it.cfg == head.cfg && it.pw == head.pw && it.cfg != CFG_128x256;
      if (b0 != a0 && (it.cfg == CFG_128x256 || head.cfg == CFG_128x256)) continue;  // fills the chip alone
      if (!same && !(mixable(head) && mixable(it))) continue;
      uniform = uniform && same;
      done[b0] = true;
      const Prepared& pr = it.pr;
      grp.first[grp.count + 1] = grp.first[grp.count] + (int)pr.grid;
      grp.p[grp.count++] = pr.prob;
      if (pr.prob.splits > 1 || pr.prob.splits < -1) {
        red.first[red.count + 1] = red.first[red.count] + (int)pr.reduce_grid;
        red.p[red.count++] = pr.red;
      }
    }
    const unsigned grid = (unsigned)grp.first[grp.count];
    if (grp.count == 1 && is_wave(head.cfg)) {
      launch_wave(head.dtype, head.pw, head.cfg, head.pr, s);
    } else if (grp.count == 1) {
      launch_single(head.dtype, head.cfg, head.pw, grid, s, grp.p[0]);
    } else if (uniform && !is_wave(head.cfg)) {
      OGLE_IGEMM_DISPATCH(conv_igemm_group_kernel, head.dtype, head.cfg, head.pw, grid, s, grp);
    } else if (head.dtype == OGLE_F16) {
      launch((conv_igemm_mixed_kernel<__half, 128>), dim3(grid), dim3(256), 0, s, grp);
    } else {
      launch((conv_igemm_mixed_kernel<float, kRowBytesF32>), dim3(grid), dim3(256), 0,
                         s, grp);
    }
    int32_t st = check_launch("conv_igemm_group");
    if (st != OGLE_OK) return st;
    if (red.count == 0 || reduce_pending != nullptr) continue;  // the caller finishes them later
    const dim3 rgrid((unsigned)red.first[red.count]), block(256);
    if (red.count == 1) {
      Prepared one{};
      one.red = red.p[0];
      one.reduce_grid = rgrid.x;
      one.reduce_lanes = red.p[0].lanes;
      if (head.dtype == OGLE_F16) launch_reduce_single<__half>(one, s);
      else launch_reduce_single<float>(one, s);
    } else if (head.dtype == OGLE_F16) {
      launch((splitk_reduce_group_kernel<__half>), rgrid, block, 0, s, red);
    } else {
      launch((splitk_reduce_group_kernel<float>), rgrid, block, 0, s, red);
    }
    st = check_launch("splitk_reduce_group");
    if (st != OGLE_OK) return st;
  }
  return OGLE_OK;
}

// Finishes convolutions whose contraction was launched with the reduction left pending:
// the plan is a function of the arguments alone, so it is recomputed here and names the
// same partial-sum layout.  All reductions go out in one grid (16 problems per grid).
int32_t launch_conv_reduce(const OgleConvArgs* args, int count, hipStream_t s) {
  int at = 0;
  while (at < count) {
    ReduceGroup red{};
    int dtype = -1;
    for (; at < count && red.count < kMaxGroup; ++at) {
      long m = 0;
      if (!igemm_eligible(args[at], &m) || f16_async_config(args[at]) >= 0) continue;
      const IgemmPlan p = final_plan(args[at], m);
      if (p.splits <= 1) continue;
      if (dtype >= 0 && args[at].dtype != dtype) break;  // one storage type per grid
      dtype = args[at].dtype;
      const Prepared pr = prepare(args[at], m, p);
      red.first[red.count + 1] = red.first[red.count] + (int)pr.reduce_grid;
      red.p[red.count++] = pr.red;
    }
    if (red.count == 0) continue;
    const dim3 rgrid((unsigned)red.first[red.count]), block(256);
    if (dtype == OGLE_F16) {
      launch((splitk_reduce_group_kernel<__half>), rgrid, block, 0, s, red);
    } else {
      launch((splitk_reduce_group_kernel<float>), rgrid, block, 0, s, red);
    }
    const int32_t st = check_launch("splitk_reduce_group");
    if (st != OGLE_OK) return st;
  }
  return OGLE_OK;
}

// ---------------------------------------------------------------------------
// Split-K scratch that lives in the library's device image, for callers that may
// not allocate.  Every GPU the library runs on holds its own copy of the array
// until the process ends.  In host code the array's name is only a stand-in for the
// symbol, not a device address: the address on the current device comes from
// hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
static __device__ __align__(256) unsigned char scratch[OGLE_CONV_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device (resolved at the first call on it).
int32_t static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("conv2d_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    return OGLE_ERR_NO_DEVICE;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    set_error("conv2d_noalloc: device ordinal %d outside 0..%d", dev, kMaxDevices - 1);
    return OGLE_ERR_UNSUPPORTED;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("conv2d_noalloc: hipGetSymbolAddress(scratch) on device %d: %s", dev,
                hipGetErrorString(e));
      return OGLE_ERR_NO_DEVICE;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return OGLE_OK;
}
}  // namespace

// launch_conv_igemm with the split-K partial sums in the static array.  The split-K
// kernels write every partial they later read, so nothing has to start at zero.
int32_t launch_conv_igemm_static_scratch(const OgleConvArgs& a, hipStream_t s) {
  long m = 0;
  if (!igemm_eligible(a, &m)) return OGLE_ERR_UNSUPPORTED;  // the other kernels use no scratch
  const size_t need = f16_async_config(a) >= 0 ? 0 : plan_igemm(a, m, true).workspace_bytes;
  if (need > (size_t)OGLE_CONV_NOALLOC_SCRATCH_BYTES) {
    set_error("conv2d_noalloc: this convolution's split-K plan needs %zu bytes of scratch, the "
              "built-in buffer holds %zu; use ogle_hip_conv2d with a caller workspace",
              need, (size_t)OGLE_CONV_NOALLOC_SCRATCH_BYTES);
    return OGLE_ERR_INVALID_ARG;
  }
  OgleConvArgs q = a;
  q.workspace_dev = nullptr;
  q.workspace_bytes = 0;
  if (need > 0) {
    void* ptr = nullptr;
    const int32_t st = static_scratch(&ptr);
    if (st != OGLE_OK) return st;
    q.workspace_dev = ptr;
    q.workspace_bytes = (size_t)OGLE_CONV_NOALLOC_SCRATCH_BYTES;
  }
  return launch_conv_igemm(q, s);
}

}  // namespace ogle
