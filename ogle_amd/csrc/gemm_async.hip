// Pointwise (1x1, stride 1, no padding) convolution with fp16 storage as a GEMM on the MFMA
// units, operands streamed global -> LDS without passing through registers
// (conv2d_pw.glsl:35-91 computes the same sums, one output texel per fragment).
//
//   Y[m, o] = act( bias[o] + sum_c X[m, c] * W[o, c] ),   m = (image, y, x) flattened
//
// Both operands are K-contiguous (NHWC activations, OHWI filter), so a tile row is a run of
// bytes along K in memory and in LDS alike.
//
// Data movement.  A K step ("stage") is 32 channels: 64 bytes of every tile row.  A wave
// fetches 1 KB of a stage with ONE buffer_load_dwordx4 ... lds instruction: lane l's 16 bytes
// land at M0 + 16 * l, i.e. the 64 lanes fill 16 consecutive LDS rows of 64 bytes.  Which
// 16-byte K group ("kvec") of its row a lane fetches is permuted so that the MFMA operand
// reads below hit every LDS bank once (slot_xor).  Rows past the end of the
// problem and K groups past the end of K are fetched at an out-of-range buffer offset, which
// writes zeros to LDS.  NST stage buffers form a ring; stage s + NST - 1 is requested right
// after the barrier that frees the buffer stage s - 1 was multiplied from, so NST - 1 stages
// are in flight while one is multiplied.  The loads are issued from inline assembly and
// counted by hand (s_waitcnt vmcnt): the compiler would otherwise wait for every outstanding
// load before the first LDS read that follows one.
//
// MFMA mapping.  v_mfma_f32_32x32x16_f16 with the filter rows as the first operand and the
// activation rows as the second: lane l supplies W[o0 + l % 32][8 * (l / 32) ..+7] and
// X[m0 + l % 32][same k], one 16-byte LDS read each, and register r of lane l then holds
// output channel o0 + 8 * (r / 4) + 4 * (l / 32) + r % 4 of pixel m0 + l % 32: four consecutive
// channels of one pixel per register quad, which the epilogue converts, packs and passes
// through LDS so that global stores are 16 bytes per lane along a pixel's channels.
//
// LDS reads.  A ds_read_b128 is served 16 lanes per cycle, and the 16 lanes that share a cycle
// are those with the same lane / 32 and the same parity of (lane >> 2) & 7 (measured on MI355X
// with pairs of lanes aimed at one bank); they must fall into 16 different 16-byte columns of a
// 256-byte window.  With 64-byte rows, slot = kvec ^ ((row >> 2) & 3) does that for the MFMA
// read pattern (row = lane % 32, kvec = 2 * chunk + lane / 32).
//
// Eight waves per workgroup, two per SIMD, in two groups that alternate between reading
// operands and issuing MFMAs (see the loop), 256 x 256 or 192 x 256 outputs per workgroup.
//
// The kernel is written for either storage type, but only fp16 storage is routed here: with
// fp32 operands (v_mfma_f32_32x32x2_f32 does a sixteenth of the work per operand byte and per
// cycle) 128 x 128 ... 256 x 256 tiles of this form measured 70-111 TFLOP/s on the network's
// pointwise layers, alone and with two or four launches in flight, against 88-115 TFLOP/s for
// the LDS-tiled kernel with its small 64 x 64 tiles, which spread far better over 256 compute
// units at those sizes.
#include "common.h"

#pragma clang diagnostic ignored "-Winline-asm"

namespace ogle {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr unsigned kOutOfRange = 0x80000000u;
constexpr int kStageRowBytes = 64;   // K bytes per tile row per stage (32 halves)

struct AsyncProblem {
  const void* x;
  const void* w;
  const float* bias;
  void* y;
  int m, n, k;             // pixels, output channels, input channels
  unsigned x_bytes, w_bytes;
  int tiles_m, tiles_n;
  long oimg;               // elements between the outputs of consecutive images; 0: dense
  int hw;                  // pixels per image
  Epilogue ep;
};

// Buffer descriptor (raw, untyped, range-checked against `bytes`) in four scalar registers.
__device__ __forceinline__ u32x4 make_desc(const void* base, unsigned bytes) {
  const unsigned long a = reinterpret_cast<unsigned long>(base);
  u32x4 d;
  d[0] = __builtin_amdgcn_readfirstlane((unsigned)a);
  d[1] = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32) & 0xffffu);
  d[2] = __builtin_amdgcn_readfirstlane(bytes);
  d[3] = 0x00020000u;
  return d;
}

// 64 lanes x 16 bytes from buffer offsets `voff` to LDS bytes [lds_addr, lds_addr + 1024).
__device__ __forceinline__ void load_to_lds(unsigned lds_addr, unsigned voff, const u32x4& desc) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(desc)
               : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_loads_outstanding() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Bank permutation of a row's four 16-byte slots: slot = kvec ^ slot_xor(row) (file comment).
__device__ __forceinline__ int slot_xor(int row) { return (row >> 2) & 3; }

template <int BM, int BN, int WM, int WN, int NST>
constexpr int async_lds_bytes() {
  constexpr int pieces = (BM + BN) * kStageRowBytes / 1024, waves = WM * WN;
  constexpr int spare = (pieces + waves - 1) / waves * waves - pieces;
  // the stage ring, then the tile's bias, then the dummy region of the spare load slots
  return NST * (BM + BN) * kStageRowBytes + BN * 4 + spare * 1024;
}

template <typename T, int BM, int BN, int WM, int WN, int NST>
__global__ __launch_bounds__(64 * WM * WN, 1) void pw_gemm_async_kernel(AsyncProblem p) {
  constexpr int NW = WM * WN;
  constexpr unsigned ESZ = sizeof(T);
  constexpr int KS = kStageRowBytes;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;       // 32x32 MFMA blocks per wave: pixels, channels
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && TM >= 1 && TN >= 1, "wave tile in whole MFMA blocks");
  constexpr int STAGE = (BM + BN) * KS;
  constexpr int CH = STAGE / 1024;                  // 1 KB pieces per stage (16 rows each)
  constexpr int CHX = BM * KS / 1024;               // of which activation rows
  static_assert(STAGE % 1024 == 0 && (BM * KS) % 1024 == 0, "operands in whole 1 KB pieces");
  // every wave issues the same number of loads per stage (the counting below relies on it):
  // when the pieces do not divide evenly, the spare slots fetch zeros into a dummy region
  constexpr int LPW = (CH + NW - 1) / NW;
  constexpr int SPARE = LPW * NW - CH;
  static_assert(LPW * (NST - 1) < 64, "outstanding loads must fit the vmcnt counter");
  static_assert(SPARE >= 0 && SPARE < NW, "spare load slots");
  static_assert(NST >= 3, "ring of at least three stages");

  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const unsigned lds_base =
      (unsigned)reinterpret_cast<unsigned long>((__attribute__((address_space(3))) unsigned char*)lds);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / WN, wave_n = wave % WN;

  // tile rows (the tiles sharing one band of activation rows) are dealt to the 8 XCDs
  const int bid = (int)blockIdx.x;
  const int xcd = bid & 7, j = bid >> 3;
  const int tile_m = (j / p.tiles_n) * 8 + xcd;
  const int tile_n = j % p.tiles_n;
  if (tile_m >= p.tiles_m) return;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const u32x4 dx = make_desc(p.x, p.x_bytes);
  const u32x4 dw = make_desc(p.w, p.w_bytes);
  const unsigned krow = (unsigned)p.k * ESZ;        // bytes per operand row

  // The pieces this wave fetches each stage: piece c = wave + NW * i covers tile rows
  // [16 c, 16 c + 16); this lane's row of it and the K group it fetches.
  unsigned g_off[LPW];    // byte offset of (row, kvec) at stage 0, or out of range
  unsigned g_kb[LPW];     // K byte of the lane's group inside a stage
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int c = wave + NW * i;
    const int row = c * 16 + (lane >> 2);
    const int kvec = (lane & 3) ^ slot_xor(row);
    g_kb[i] = (unsigned)kvec * 16u;
    if (c < CHX) {
      const int m = m0 + row;
      g_off[i] = m < p.m ? (unsigned)m * krow + g_kb[i] : kOutOfRange;
    } else if (c < CH) {
      const int o = n0 + row - BM;
      g_off[i] = o < p.n ? (unsigned)o * krow + g_kb[i] : kOutOfRange;
    } else {
      g_off[i] = kOutOfRange;   // a spare slot
    }
  }
  const int stages = (int)((krow + KS - 1) / KS);

  auto request_stage = [&](int s) {
    const unsigned kb = (unsigned)s * KS;
    const unsigned buf = lds_base + (unsigned)(s % NST) * STAGE;
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int c = wave + NW * i;
      const bool ok = g_off[i] != kOutOfRange && kb + g_kb[i] < krow;
      const unsigned voff = ok ? g_off[i] + kb : kOutOfRange;
      // the piece's operand: a scalar choice (c is the same for the whole wave)
      u32x4 d;
#pragma unroll
      for (int e = 0; e < 4; ++e) d[e] = c < CHX ? dx[e] : dw[e];
      const unsigned dst = c < CH ? buf + (unsigned)c * 1024u
                                  : lds_base + (unsigned)(NST * STAGE + BN * 4 + (c - CH) * 1024);
      load_to_lds(dst, voff, d);
    }
  };

  // operand reads: lane l reads row l % 32 of a block, K group 2 * chunk + l / 32
  const int l32 = lane & 31, lh = lane >> 5;
  const int sx = slot_xor(l32);
  const unsigned rd_x = (unsigned)((wave_m * WTM + l32) * KS);
  const unsigned rd_w = (unsigned)((BM + wave_n * WTN + l32) * KS);
  const unsigned rd_k[2] = {(unsigned)(((0 + lh) ^ sx) * 16), (unsigned)(((2 + lh) ^ sx) * 16)};

  floatx16 acc[TN][TM];
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // Two groups of waves (see the loop below).  Group 1 requests NST - 1 stages ahead of the
  // one it reads, group 0 one stage less.
  static_assert(NST >= 4 && NW % 2 == 0, "ping-pong needs two wave groups and four stages");
  const int grp = wave / (NW / 2);
#pragma unroll
  for (int s = 0; s < NST - 2; ++s) request_stage(s);
  if (grp == 1) request_stage(NST - 2);

  // the tile's bias values wait in LDS behind the stage ring for the epilogue
  float* const bias_lds = reinterpret_cast<float*>(lds + NST * STAGE);
  if (tid < BN / 4) {
    const int o = n0 + tid * 4;
    float4 bv = make_float4(0.f, 0.f, 0.f, 0.f);
    if (p.bias != nullptr && o < p.n) bv = *reinterpret_cast<const float4*>(p.bias + o);
    *reinterpret_cast<float4*>(bias_lds + tid * 4) = bv;
  }

  u32x4 xv[2][TM], wv[2][TN];
  auto read_stage = [&](int s) {
    const unsigned char* buf = lds + (s % NST) * STAGE;
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
#pragma unroll
      for (int b = 0; b < TM; ++b)
        xv[ch][b] = *reinterpret_cast<const u32x4*>(buf + rd_x + b * 32 * KS + rd_k[ch]);
#pragma unroll
      for (int a = 0; a < TN; ++a)
        wv[ch][a] = *reinterpret_cast<const u32x4*>(buf + rd_w + a * 32 * KS + rd_k[ch]);
    }
  };
  // fp16: a lane's 16 bytes are the 8 halves one v_mfma_f32_32x32x16_f16 wants (k = 8 * (l / 32) ..+7).
  // fp32: they are 4 floats, one v_mfma_f32_32x32x2_f32 each (the contraction sums over k in any
  // order: lanes 0-31 supply k 0..3 of an 8-wide group, lanes 32-63 k 4..7).
  auto multiply_stage = [&]() {
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
      if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
          for (int b = 0; b < TM; ++b)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, wv[ch][a]),
                                                               __builtin_bit_cast(halfx8, xv[ch][b]),
                                                               acc[a][b], 0, 0, 0);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b)
              acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(wv[ch][a][e]),
                                                               __uint_as_float(xv[ch][b][e]), acc[a][b], 0, 0, 0);
      }
    }
  };
  // A barrier without the fence of __syncthreads(): it waits for no memory operation of the
  // wave, so operand reads issued before it may still be in flight behind it.  Neither the
  // compiler nor the instruction scheduler moves anything across it.
#define OGLE_PHASE_BARRIER()              \
  __builtin_amdgcn_sched_barrier(0);      \
  asm volatile("" ::: "memory");          \
  __builtin_amdgcn_s_barrier();           \
  asm volatile("" ::: "memory");          \
  __builtin_amdgcn_sched_barrier(0)

  // Two groups of waves, one wave of each on every SIMD, take turns: while one group reads
  // its operands of a stage from LDS and requests a further stage ("memory phase"), the
  // other issues the MFMAs of the stage it read before ("compute phase"); a barrier ends
  // every phase.  Group 1 runs one phase behind group 0:
  //   phase      2s      2s+1    2s+2
  //   group 0:   M(s)    C(s)    M(s+1)
  //   group 1:   C(s-1)  M(s)    C(s)
  // The barriers do not wait for the LDS reads of a memory phase: their data arrive while the
  // first MFMAs of the compute phase that follows are issued (every value read is consumed
  // by an MFMA of that phase, so at its end the reads are complete).  What keeps the ring
  // consistent:
  //  - a stage is read after it has landed: before the barrier that ends phase 2s - 1 every
  //    wave waits for its own pieces of stage s, which group 0 reads in phase 2s and group 1
  //    in phase 2s + 1;
  //  - a buffer is overwritten after it has been read: stage s has been read completely at
  //    the end of phase 2s + 1 by group 0 and of phase 2s + 2 by group 1, so the request that
  //    reuses its buffer (for stage s + NST) is issued in phase 2s + 3 or later: group 1 does
  //    that in M(s + 1), i.e. it requests NST - 1 stages ahead; group 0's first memory phase
  //    late enough is M(s + 2), so it requests NST - 2 stages ahead.
  if (grp == 0) {
    wait_loads_outstanding<LPW * (NST - 3)>();   // own pieces of stage 0
  } else {
    wait_loads_outstanding<LPW * (NST - 2)>();   // the same, with one more stage in flight
  }
  OGLE_PHASE_BARRIER();
  if (grp == 0) {
    for (int s = 0; s < stages; ++s) {
      read_stage(s);
      request_stage(s + NST - 2);
      OGLE_PHASE_BARRIER();
      multiply_stage();
      wait_loads_outstanding<LPW * (NST - 3)>();   // own pieces of stage s + 1
      OGLE_PHASE_BARRIER();
    }
  } else {
    OGLE_PHASE_BARRIER();
    for (int s = 0; s < stages; ++s) {
      read_stage(s);
      request_stage(s + NST - 1);
      wait_loads_outstanding<LPW * (NST - 2)>();   // own pieces of stage s + 1
      OGLE_PHASE_BARRIER();
      multiply_stage();
      if (s + 1 < stages) { OGLE_PHASE_BARRIER(); }
    }
  }
#undef OGLE_PHASE_BARRIER
  // the zero-filled requests past the last stage still write LDS: they must have landed
  // before this wave ends and its workgroup's LDS can be handed to another one
  wait_loads_outstanding<0>();

  // Epilogue.  A lane holds four consecutive channels of one pixel per register quad; stored
  // straight from there every lane would write 8 bytes to a row of its own (64 requests per
  // instruction, and the L2 takes one request per cycle and channel whatever its size).  So a
  // wave passes each block of 32 pixels through a private LDS region: bias, activation and
  // conversion on the way in (8 bytes per quad), 16 bytes per lane on the way out with
  // consecutive lanes on consecutive channels of one pixel, i.e. whole 128-byte runs per row.
  __syncthreads();   // every wave has finished reading the stage buffers that are reused here
  constexpr int ROWP = WTN * (int)ESZ + 16;     // staged row: the wave's channels in storage type, padded
  constexpr int SEGS = WTN * (int)ESZ / 16;     // 16-byte segments (lanes) per row
  constexpr int RPI = 64 / SEGS;                // rows one store instruction covers
  constexpr int EPS = 16 / (int)ESZ;            // elements per 16-byte segment
  static_assert(NW * 32 * ROWP <= NST * STAGE, "epilogue staging exceeds the stage buffers");
  static_assert(SEGS <= 64 && 64 % SEGS == 0 && 32 % RPI == 0, "staged rows divide among the lanes");
  unsigned char* const stg = lds + wave * (32 * ROWP);
  T* const y = static_cast<T*>(p.y);
  const int seg = lane % SEGS, rsub = lane / SEGS;
  const int ocol = n0 + wave_n * WTN + seg * EPS;
#pragma unroll
  for (int b = 0; b < TM; ++b) {
#pragma unroll
    for (int a = 0; a < TN; ++a) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int oc = a * 32 + q * 8 + lh * 4;   // channel inside the wave's tile
        const float4 bv = *reinterpret_cast<const float4*>(bias_lds + wave_n * WTN + oc);
        const float o0 = apply_epilogue(acc[a][b][q * 4 + 0] + bv.x, p.ep);
        const float o1 = apply_epilogue(acc[a][b][q * 4 + 1] + bv.y, p.ep);
        const float o2 = apply_epilogue(acc[a][b][q * 4 + 2] + bv.z, p.ep);
        const float o3 = apply_epilogue(acc[a][b][q * 4 + 3] + bv.w, p.ep);
        if constexpr (sizeof(T) == 2) {
          halfx4 out;
          out[0] = (_Float16)o0; out[1] = (_Float16)o1; out[2] = (_Float16)o2; out[3] = (_Float16)o3;
          *reinterpret_cast<halfx4*>(stg + l32 * ROWP + oc * 2) = out;
        } else {
          *reinterpret_cast<float4*>(stg + l32 * ROWP + oc * 4) = make_float4(o0, o1, o2, o3);
        }
      }
    }
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const int row = it * RPI + rsub;
      const u32x4 v = *reinterpret_cast<const u32x4*>(stg + row * ROWP + seg * 16);
      const int m = m0 + wave_m * WTM + b * 32 + row;
      if (m < p.m && ocol < p.n) {
        long row_at;
        if (p.oimg == 0) {
          row_at = (long)m * p.n;
        } else {
          const int img = m / p.hw;
          row_at = (long)img * p.oimg + (long)(m - img * p.hw) * p.n;
        }
        store_result16(y + row_at + ocol, make_uint4(v[0], v[1], v[2], v[3]));
      }
    }
  }
}

enum { kTile256 = 0, kTile192 = 1 };   // 256 x 256 or 192 x 256 outputs per workgroup

template <typename T, int BM, int BN, int WM, int WN, int NST>
int32_t launch_tile(AsyncProblem p, hipStream_t s) {
  constexpr int kLds = async_lds_bytes<BM, BN, WM, WN, NST>();
  auto kernel = pw_gemm_async_kernel<T, BM, BN, WM, WN, NST>;
  // more than 64 KB of dynamic LDS has to be asked for once per device and kernel
  static bool configured[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    set_error("pw_gemm_async: no current device");
    return OGLE_ERR_NO_DEVICE;
  }
  if (!configured[dev]) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) {
      set_error("pw_gemm_async: cannot reserve %d bytes of LDS: %s", kLds, hipGetErrorString(e));
      return OGLE_ERR_LAUNCH;
    }
    configured[dev] = true;
  }
  p.tiles_m = (p.m + BM - 1) / BM;
  p.tiles_n = (p.n + BN - 1) / BN;
  const unsigned grid = 8u * (unsigned)((p.tiles_m + 7) / 8) * (unsigned)p.tiles_n;
  launch(kernel, dim3(grid), dim3(64 * WM * WN), (unsigned)kLds, s, p);
  return check_launch("pw_gemm_async");
}

}  // namespace

// The shapes the kernel above takes: fp16 storage, pointwise, one destination, channel counts
// that keep every 16-byte K group and every 8-byte store whole, and enough rows to fill tiles.
int f16_async_config(const OgleConvArgs& a) {
  if (a.dtype != OGLE_F16 || a.group != 1) return -1;
  if (a.kernel_size != 1 || a.stride != 1 || a.padding != 0) return -1;
  if (a.output2_dev != nullptr) return -1;
  if (a.in_c % 8 != 0 || a.out_c % 8 != 0) return -1;
  if ((a.out_image_stride & 7) != 0) return -1;
  const long m = (long)a.n * a.out_h * a.out_w;
  // measured on MI355X against the LDS-tiled kernel: it pays with at least 256 input
  // channels (fewer: the launch is over before the ring has filled) and when the 256-wide
  // tile columns are at least three quarters full
  if (m < 2048 || a.in_c < 256) return -1;
  if (a.out_c * 4 < ((a.out_c + 255) / 256) * 256 * 3) return -1;
  if (m * a.in_c * 2 > 0x7fffffffL || (long)a.out_c * a.in_c * 2 > 0x7fffffffL) return -1;
  // 256 x 256 tiles or 192 x 256 tiles, whichever needs less MFMA time on the busiest of the
  // 256 compute units (rounds of tiles x tile area); the larger tile on a tie (it pulls less
  // from L2).  With fewer than half the units busy the LDS-tiled kernel is the better choice.
  const long tn = (a.out_c + 255) / 256;
  const long t256 = ((m + 255) / 256) * tn, t192 = ((m + 191) / 192) * tn;
  const long c256 = ((t256 + 255) / 256) * 256 * 256, c192 = ((t192 + 255) / 256) * 192 * 256;
  if (c192 < c256) return t192 >= 128 ? kTile192 : -1;
  return t256 >= 128 ? kTile256 : -1;
}

int32_t launch_pw_gemm_f16_async(const OgleConvArgs& a, hipStream_t s) {
  const int cfg = f16_async_config(a);
  if (cfg < 0) return OGLE_ERR_UNSUPPORTED;
    AsyncProblem p{};
  p.x = a.input_dev;
  p.w = a.filter_dev;
  p.bias = a.bias_dev;
  p.y = a.output_dev;
  p.m = (int)((long)a.n * a.out_h * a.out_w);
  p.n = a.out_c;
  p.k = a.in_c;
  const long esz = a.dtype == OGLE_F16 ? 2 : 4;
  p.x_bytes = (unsigned)((long)p.m * p.k * esz);
  p.w_bytes = (unsigned)((long)p.n * p.k * esz);
  p.hw = a.out_h * a.out_w;
  p.oimg = a.out_image_stride == (long)p.hw * a.out_c ? 0 : a.out_image_stride;
  p.ep = make_epilogue(a.act, a.min_value, a.max_value, a.act_variant);
  switch (cfg) {
    case kTile192: return launch_tile<__half, 192, 256, 2, 4, 4>(p, s);
    case kTile256: return launch_tile<__half, 256, 256, 2, 4, 4>(p, s);
    default: return OGLE_ERR_UNSUPPORTED;
  }
}

}  // namespace ogle
