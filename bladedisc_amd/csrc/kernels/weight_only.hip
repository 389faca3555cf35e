// Weight-only quantized GEMM for gfx950: floating-point activations (f16 or f32) times 8-bit
// weights with a per-output-channel scale and zero point,
//
//   out[m, n] = (sum_k x[m, k] * (w[n, k] - zp[n])) * scale[n] + bias[n]
//
// which is matmul(x, dequantize(w)^T) + bias with the scale taken out of the sum.  This is the
// runtime side of the reference's `ral_pdll_weight_only_qgemm` custom call
// (pytorch_blade/tests/disc/pdl/pdll_files/gpu/weight_only_qgemm.pdll:2-104; operands input,
// weight ui8 [K, N], [bias,] weight_scale, weight_zero_point), for which the reference tree
// holds no implementation.
//
// The weights stay 8-bit in memory and are widened on their way into the matrix cores
// (v_mfma_f32_32x32x16_f16, f32 accumulation): a byte b becomes the half 0x6400 | b = 1024 + b
// with one v_perm_b32 per two weights, and one packed subtraction of 1024 + zp[n] leaves
// b - zp[n] exactly (|b - zp| <= 2048 is an integer a half holds).  Products of a half
// activation (11 significant bits) and such a weight (9 bits) are exact in f32, so the only
// rounding is the f32 accumulation.  f32 activations are split into two halves
// x = hi + lo (hi = half(x), lo = half(x - hi)) and both are multiplied: about 22 significant
// bits of x take part while lo is a normal half (|x| >= 1/8); below, lo is subnormal and the
// error per activation is an absolute 2^-25.
//
// In the register kernels both operands go from global memory straight into registers in MFMA
// layout: the order of the k values inside a fragment is free as long as both operands agree,
// so lane (row, g) takes the 16 consecutive k values k0 + 16 g .. of its row -- 16 weight bytes
// (one dwordx4), 16 activations -- and feeds two MFMAs with them.
//  * wo_lds_kernel: tiles shared through LDS, everything above 32 rows (16 for f32): 64 x 64 or 128 x 128
//    tiles while the problem is a few rounds of them -- with several workgroups per tile, each
//    over a part of k, and wo_splitk_reduce_kernel behind them, where that is estimated
//    cheaper --, 256 x 128 and 256 x 256 tiles beyond (1.06-1.16 PFLOP/s for f16 activations
//    at 4096^2 .. 8192^2 weights, where the ROCm library's plain f16 GEMM reaches 1.16-1.49);
//  * wo_tile_kernel: 2 x 2 waves, wave tile (32 FM) x (32 FN), operands straight into registers:
//    operands too large for the LDS kernel's 31-bit offsets;
//  * wo_skinny_lds_kernel: 5 .. 32 rows (16 for f32 activations) against deep or wide weights,
//    32 output channels per workgroup, both operands loaded in row segments and turned into
//    fragments through wave-private LDS;
//  * wo_gemv_kernel: one or two rows, a wave per output channel streaming its weight row on the
//    vector ALUs;
//  * wo_skinny16_kernel: M <= 16 rows against 16 output channels per workgroup (16x16x32 MFMA);
//  * wo_skinny_kernel: M <= 128 rows against 32 output channels per workgroup, the k range dealt
//    over the waves and the partial sums added through LDS (bound by the weight bytes: 1 byte
//    per weight from HBM);
//  * wo_generic_kernel: one output per thread, any layout and alignment (also weights left as
//    [K, N]).
#include <algorithm>

#include "dq8_common.h"
#include "disc_q8.h"

#pragma clang fp contract(off)

namespace dq8 {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));

// gfx9 raw buffer descriptor word 3: 32-bit data format, no swizzle
constexpr int kBufferWord3 = 0x00020000;

struct WoParams {
  const void* x;        // [M, K] activations, row stride ldx elements
  const uint8_t* w;     // weights; element (n, k) at w[n * w_sn + k * w_sk]
  const void* scale;    // [N], activation dtype
  const int32_t* zp;    // [N] or null (zero)
  const void* bias;     // [N] or null, activation dtype
  void* out;            // [M, N], row stride ldo elements
  int64_t ldx, ldo, w_sn, w_sk;
  int M, N, K;
  unsigned flip;        // 0x80808080 for signed weights (b ^ 0x80 = b + 128 as unsigned)
  // split k (wo_lds_kernel): workgroup (tile, y) multiplies k in [y k_split, (y + 1) k_split)
  // and, when `partial` is set, leaves its f32 sums in partial[y][M][N] for the reduction kernel
  float* partial;
  int k_split;          // a multiple of 64; K when the k range is not split
};

template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return (float)v;
}

// 16 weight bytes -> the halves of two MFMA k-steps, minus c = 1024 + zp (+128 if signed)
__device__ __forceinline__ void widen16(u4 q, unsigned flip, h2 c, h8& s0, h8& s1) {
  auto pair = [&](unsigned d, unsigned sel) {
    return __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, d ^ flip, sel)) - c;
  };
  const h2 a0 = pair(q.x, 0x05010400u), a1 = pair(q.x, 0x07030602u);
  const h2 a2 = pair(q.y, 0x05010400u), a3 = pair(q.y, 0x07030602u);
  const h2 b0 = pair(q.z, 0x05010400u), b1 = pair(q.z, 0x07030602u);
  const h2 b2 = pair(q.w, 0x05010400u), b3 = pair(q.w, 0x07030602u);
  s0 = (h8){a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
  s1 = (h8){b0.x, b0.y, b1.x, b1.y, b2.x, b2.y, b3.x, b3.y};
}

// The 16 activations of a lane for one 32-deep k chunk: two k-steps, and for f32 activations a
// second pair holding what the first rounded away.
template <typename XT>
struct XFrag;

template <>
struct XFrag<_Float16> {
  u4 r0, r1;
  static constexpr int kParts = 1;
  __device__ __forceinline__ void load(const _Float16* p, bool valid) {
    const u4 z = {0, 0, 0, 0};
    r0 = valid ? *reinterpret_cast<const u4*>(p) : z;
    r1 = valid ? *reinterpret_cast<const u4*>(p + 8) : z;
  }
  __device__ __forceinline__ h8 step(int part, int s) const {
    (void)part;
    return __builtin_bit_cast(h8, s == 0 ? r0 : r1);
  }
};

template <>
struct XFrag<float> {
  f4 r[4];
  static constexpr int kParts = 2;
  __device__ __forceinline__ void load(const float* p, bool valid) {
    const f4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = valid ? *reinterpret_cast<const f4*>(p + 4 * i) : z;
  }
  __device__ __forceinline__ h8 step(int part, int s) const {
    h8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = r[2 * s + e / 4][e % 4];
      const _Float16 hi = (_Float16)v;
      o[e] = part == 0 ? hi : (_Float16)(v - (float)hi);
    }
    return o;
  }
};

template <typename XT>
__device__ __forceinline__ void store_frag(const WoParams& p, const f16v& acc, int m_base, int n,
                                           int lane) {
  if (n >= p.N) return;
  const XT* scale = static_cast<const XT*>(p.scale);
  const XT* bias = static_cast<const XT*>(p.bias);
  const float s = to_f32(scale[n]);
  const float b = bias ? to_f32(bias[n]) : 0.0f;
  XT* out = static_cast<XT*>(p.out);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int m = m_base + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
    if (m < p.M) out[(int64_t)m * p.ldo + n] = (XT)(acc[v] * s + b);
  }
}

// The raw sums of one k range, for wo_splitk_reduce_kernel.
__device__ __forceinline__ void store_partial(const WoParams& p, const f16v& acc, int split,
                                              int m_base, int n, int lane) {
  if (n >= p.N) return;
  float* dst = p.partial + (int64_t)split * p.M * p.N;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int m = m_base + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
    if (m < p.M) dst[(int64_t)m * p.N + n] = acc[v];
  }
}

__device__ __forceinline__ h2 centre(const WoParams& p, int n) {
  const int zp = p.zp ? p.zp[n] : 0;
  const _Float16 c = (_Float16)(float)(1024 + zp + (p.flip ? 128 : 0));
  return (h2){c, c};
}

// ---------------------------------------------------------------- tiled kernel, M > 32
template <typename XT, int FM, int FN>
__global__ void __launch_bounds__(256) wo_tile_kernel(const WoParams p) {
  constexpr int BM = 2 * FM * 32, BN = 2 * FN * 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.N + BN - 1) / BN;
  const int m0 = (blockIdx.x / tiles_n) * BM + wm * FM * 32;
  const int n0 = (blockIdx.x % tiles_n) * BN + wn * FN * 32;
  const int r = lane & 31, g = lane >> 5;

  const XT* xrow[FM];
  const uint8_t* wrow[FN];
  h2 c[FN];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int m = min(m0 + i * 32 + r, p.M - 1);          // rows past M re-read the last one
    xrow[i] = static_cast<const XT*>(p.x) + (int64_t)m * p.ldx + 16 * g;
  }
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    const int n = min(n0 + j * 32 + r, p.N - 1);
    wrow[j] = p.w + (int64_t)n * p.w_sn + 16 * g;
    c[j] = centre(p, n);
  }
  f16v acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // D chunks of 32 in flight per wave (registers permitting: f32 activations take twice the
  // registers of f16 ones)
  constexpr int D = sizeof(XT) == 2 ? 4 : 2;
  XFrag<XT> xr[D][FM];
  u4 wr[D][FN];
  const u4 zero = {0, 0, 0, 0};
  auto load = [&](XFrag<XT>* xf, u4* wf, int k0) {
    const bool valid = k0 + 16 * g < p.K;                // K % 16 == 0: whole 16-chunks
    const int k = valid ? k0 : 0;
#pragma unroll
    for (int i = 0; i < FM; ++i) xf[i].load(xrow[i] + k, valid);
#pragma unroll
    for (int j = 0; j < FN; ++j) wf[j] = valid ? *reinterpret_cast<const u4*>(wrow[j] + k) : zero;
  };
  auto compute = [&](const XFrag<XT>* xf, const u4* wf) {
    h8 w0[FN], w1[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) widen16(wf[j], p.flip, c[j], w0[j], w1[j]);
#pragma unroll
    for (int part = 0; part < XFrag<XT>::kParts; ++part)
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const h8 a0 = xf[i].step(part, 0), a1 = xf[i].step(part, 1);
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, w0[j], acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, w1[j], acc[i][j], 0, 0, 0);
        }
      }
  };
  // a ring of D chunks: each is multiplied and at once refilled with the chunk D further on,
  // so D - 1 loads stay in flight under every multiplication (one chunk ahead measured 16 % of
  // the matrix rate: a wave waited out the whole load latency per chunk)
#pragma unroll
  for (int d = 0; d < D; ++d) load(xr[d], wr[d], d * 32);
  for (int k0 = 0; k0 < p.K; k0 += D * 32) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      compute(xr[d], wr[d]);
      load(xr[d], wr[d], k0 + (D + d) * 32);             // (past K: zeros)
    }
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
      store_frag<XT>(p, acc[i][j], m0 + i * 32, n0 + j * 32 + r, lane);
}

// ---------------------------------------------------------------- tiled kernel through LDS (f16)
// (64 WM) x 128 tile, WM x 2 waves (WM = 1, 2 or 4), k tiles of 64 in two LDS stages.  The
// register kernel above makes every lane fetch its own row, 64 cache lines per load
// instruction, and the compute unit's address path caps it at about 15 bytes per clock
// (0.4 PFLOP/s whatever the shape); here eight lanes cover one 128-byte row segment of the
// activations and four one 64-byte segment of the weights, the tile is shared through LDS
// (16-byte chunks XOR-swizzled by the row so that the fragment reads spread over the banks),
// and the fragments are read back as ds_read_b128.  The weights are widened to halves once,
// on their way into LDS (128-byte rows like the activations'), not by every wave that reads
// them.
//
// Four register sets hold the k tiles t + 1 .. t + 4 on their way from memory while tile t is
// multiplied.  The loads are buffer loads without a branch around them (a chunk past the k
// range gets an offset past the descriptor and reads zeros) and the main loop is four k tiles
// of straight-line code, so that the wait in front of a tile's hand-over to LDS counts the
// loads issued after it instead of draining them all: with conditional loads in a loop of
// guarded steps every k tile waited out a whole trip to memory (0.8 us per k tile on a
// quiet chip, 1.5-2 us on a busy one).
//
// f32 activations (XT = float) are split on their way into LDS, x = hi + lo with hi = half(x)
// and lo = half(x - hi), into two half tiles of the same layout; every weight fragment is
// multiplied with both.
template <typename XT, int WM, int FM, int FN, int SETS>
__global__ void __launch_bounds__(WM * 128, (WM == 1 || sizeof(XT) == 4) ? 1 : 2)
    wo_lds_kernel(const WoParams p) {
  constexpr bool F32 = sizeof(XT) == 4;
  constexpr int BM = WM * FM * 32, BN = 2 * FN * 32, BK = 64;
  constexpr int NT = WM * 128;                           // WM x 2 waves
  constexpr int XL = F32 ? 16 : 8;                       // lanes (16 bytes each) per activation row
  constexpr int XP = (BM * XL) / NT;                     // activation chunks per thread
  constexpr int WP = (BN * 4) / NT;                      // weight chunks per thread
  constexpr int XS = BM * 128 * (F32 ? 2 : 1);           // activation bytes of a stage
  constexpr int kPast = (int)0x80000000;                 // an offset no descriptor covers
  static_assert(SETS % 2 == 0 && SETS * (XP + WP) <= 63, "two LDS stages; vmcnt has 6 bits");
  // two stages of (activation tile [hi, then lo], widened weight tile), 128 bytes per row
  extern __shared__ __attribute__((aligned(16))) uint8_t wo_lds[];
  uint8_t* const xs[2] = {wo_lds, wo_lds + XS};
  uint8_t* const ws[2] = {wo_lds + 2 * XS, wo_lds + 2 * XS + BN * 128};
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.N + BN - 1) / BN;
  // Workgroups go to the 8 XCDs round-robin, and each XCD has its own L2.  Where the tile grid
  // divides, XCD x takes one compact patch of it (the grid cut 4 x 2: an activation row is
  // twice the bytes of a weight row), so that its L2 fetches the patch's operand rows instead
  // of every activation row (measured at 4096^3: 295 MB fetched per launch without this).
  int tile = blockIdx.x;
  {
    const int tiles_m = gridDim.x / tiles_n;
    // (launches of at least a round; the rows of a split launch are not dealt this way)
    if (gridDim.y == 1 && gridDim.x >= 128 && tiles_m % 4 == 0 && tiles_n % 2 == 0) {
      const int xcd = tile & 7, idx = tile >> 3;
      const int pm = tiles_m / 4, pn = tiles_n / 2;        // the patch
      tile = ((xcd >> 1) * pm + idx / pn) * tiles_n + (xcd & 1) * pn + idx % pn;
    }
  }
  const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN;
  const int r = lane & 31, g = lane >> 5;
  const int kbeg = blockIdx.y * p.k_split;               // this workgroup's k range
  const int klen = min(p.K, kbeg + p.k_split) - kbeg;
  // descriptors over the tile's rows from (first row, kbeg); the host has checked that the
  // offsets below fit 31 bits
  const int mrows = min(BM, p.M - m0), nrows = min(BN, p.N - n0);
  const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<XT*>(static_cast<const XT*>(p.x) + (int64_t)m0 * p.ldx + kbeg), 0,
      (int)(((int64_t)(mrows - 1) * p.ldx + klen) * sizeof(XT)), kBufferWord3);
  const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(p.w + (int64_t)n0 * p.w_sn + kbeg), 0,
      (int)((int64_t)(nrows - 1) * p.w_sn + klen), kBufferWord3);

  // global -> LDS assignment (rows past the tile's last re-read that one)
  const int xc = tid & (XL - 1), wc = tid & 3;           // 16-byte chunk of the row's k tile
  int xo[XP], xl[XP];
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const int row = tid / XL + (NT / XL) * i;
    const int sx = (row ^ (row >> 3)) & 7;
    xo[i] = (int)((int64_t)min(row, mrows - 1) * p.ldx * sizeof(XT)) + 16 * xc;
    // (four floats become four halves: half of the 16-byte chunk xc / 2)
    xl[i] = F32 ? row * 128 + (((xc >> 1) ^ sx) << 4) + 8 * (xc & 1)
                : row * 128 + ((xc ^ sx) << 4);
  }
  int wo[WP], wl[WP], wl1[WP];
  h2 cpark[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int row = (tid >> 2) + (NT / 4) * i;
    const int sw = (row ^ (row >> 3)) & 7;
    wo[i] = (int)((int64_t)min(row, nrows - 1) * p.w_sn) + 16 * wc;
    wl[i] = row * 128 + (((2 * wc) ^ sw) << 4);
    wl1[i] = row * 128 + (((2 * wc + 1) ^ sw) << 4);
    cpark[i] = centre(p, n0 + min(row, nrows - 1));
  }
  u4 xr[SETS][XP], wr[SETS][WP];
  auto fetch = [&](u4* xq, u4* wq, int k0) {
    const bool xv = k0 + (F32 ? 4 : 8) * xc < klen, wv = k0 + 16 * wc < klen;   // K % 16 == 0
#pragma unroll
    for (int i = 0; i < XP; ++i)
      xq[i] = __builtin_amdgcn_raw_buffer_load_b128(
          xrs, xv ? xo[i] + (int)sizeof(XT) * k0 : kPast, 0, 0);
#pragma unroll
    for (int i = 0; i < WP; ++i)
      wq[i] = __builtin_amdgcn_raw_buffer_load_b128(wrs, wv ? wo[i] + k0 : kPast, 0, 0);
  };
  auto park = [&](const u4* xq, const u4* wq, int stage) {
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      if constexpr (F32) {
        const f4 v = __builtin_bit_cast(f4, xq[i]);
        h4 hi, lo;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          hi[e] = (_Float16)v[e];
          lo[e] = (_Float16)(v[e] - (float)hi[e]);
        }
        *reinterpret_cast<h4*>(&xs[stage][xl[i]]) = hi;
        *reinterpret_cast<h4*>(&xs[stage][BM * 128 + xl[i]]) = lo;
      } else {
        *reinterpret_cast<u4*>(&xs[stage][xl[i]]) = xq[i];
      }
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      h8 lo, hi;
      widen16(wq[i], p.flip, cpark[i], lo, hi);
      *reinterpret_cast<h8*>(&ws[stage][wl[i]]) = lo;
      *reinterpret_cast<h8*>(&ws[stage][wl1[i]]) = hi;
    }
  };

  // fragment rows of this wave
  int xrow[FM], wrow[FN];
#pragma unroll
  for (int i = 0; i < FM; ++i) xrow[i] = (wm * FM + i) * 32 + r;
#pragma unroll
  for (int j = 0; j < FN; ++j) wrow[j] = (wn * FN + j) * 32 + r;
  f16v acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // (Reading the fragments of one 16-deep k step under the MFMAs of the step before, one LDS
  // read scheduled between every two MFMAs, changed nothing measurable: 135.2 against 137.5 us
  // at 4096^3 on 256 x 256 tiles.)
  auto multiply = [&](int st) {
    if constexpr (FM * FN >= 8) {
      // eight fragments per wave: one 16-deep k step at a time (this lane's 8 halves are chunk
      // 4 (q / 2) + 2 g + q % 2), the registers do not hold more fragments than that
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        h8 a[FM], al[FM], w[FN];
        const int c = 4 * (q >> 1) + 2 * g + (q & 1);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const int row = xrow[i], sx = (row ^ (row >> 3)) & 7;
          a[i] = *reinterpret_cast<const h8*>(&xs[st][row * 128 + ((c ^ sx) << 4)]);
          if constexpr (F32)
            al[i] = *reinterpret_cast<const h8*>(&xs[st][BM * 128 + row * 128 + ((c ^ sx) << 4)]);
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int row = wrow[j], sw = (row ^ (row >> 3)) & 7;
          w[j] = *reinterpret_cast<const h8*>(&ws[st][row * 128 + ((c ^ sw) << 4)]);
        }
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], w[j], acc[i][j], 0, 0, 0);
            if constexpr (F32)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[i], w[j], acc[i][j], 0, 0, 0);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
      return;
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      h8 a0[FM], a1[FM], l0[FM], l1[FM], w0[FN], w1[FN];
      const int c0 = 4 * s + 2 * g;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const int row = xrow[i], sx = (row ^ (row >> 3)) & 7;
        a0[i] = *reinterpret_cast<const h8*>(&xs[st][row * 128 + ((c0 ^ sx) << 4)]);
        a1[i] = *reinterpret_cast<const h8*>(&xs[st][row * 128 + (((c0 + 1) ^ sx) << 4)]);
        if constexpr (F32) {
          l0[i] = *reinterpret_cast<const h8*>(&xs[st][BM * 128 + row * 128 + ((c0 ^ sx) << 4)]);
          l1[i] =
              *reinterpret_cast<const h8*>(&xs[st][BM * 128 + row * 128 + (((c0 + 1) ^ sx) << 4)]);
        }
      }
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int row = wrow[j], sw = (row ^ (row >> 3)) & 7;
        w0[j] = *reinterpret_cast<const h8*>(&ws[st][row * 128 + ((c0 ^ sw) << 4)]);
        w1[j] = *reinterpret_cast<const h8*>(&ws[st][row * 128 + (((c0 + 1) ^ sw) << 4)]);
      }
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0[i], w0[j], acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1[i], w1[j], acc[i][j], 0, 0, 0);
          if constexpr (F32) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(l0[i], w0[j], acc[i][j], 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(l1[i], w1[j], acc[i][j], 0, 0, 0);
          }
        }
    }
  };
  // k tile t: set u = t % SETS has been handed to LDS stage t % 2 and takes tile t + SETS;
  // tile t + 1 (zeros past the last) is handed over behind the multiplication
  // (the scheduling barriers keep a later step's arithmetic on loaded registers -- the first
  // instructions of widening -- from being moved up to where it would wait for their loads)
  auto step = [&](int u, int t) {
    fetch(xr[u], wr[u], (t + SETS) * BK);
    multiply(u % 2);
    __builtin_amdgcn_sched_barrier(0);
    park(xr[(u + 1) % SETS], wr[(u + 1) % SETS], (u + 1) % 2);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };
  const int KT = (klen + BK - 1) / BK;
#pragma unroll
  for (int d = 0; d < SETS; ++d) fetch(xr[d], wr[d], d * BK);
  __builtin_amdgcn_sched_barrier(0);
  park(xr[0], wr[0], 0);
  __syncthreads();
  __builtin_amdgcn_sched_barrier(0);
  int t = 0;
  for (; t + SETS <= KT; t += SETS) {
#pragma unroll
    for (int u = 0; u < SETS; ++u) step(u, t + u);
  }
#pragma unroll
  for (int u = 0; u < SETS - 1; ++u)
    if (t + u < KT) step(u, t + u);                        // (uniform over the workgroup)
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
      if (p.partial)
        store_partial(p, acc[i][j], blockIdx.y, m0 + xrow[i] - r, n0 + wrow[j], lane);
      else
        store_frag<XT>(p, acc[i][j], m0 + xrow[i] - r, n0 + wrow[j], lane);
}

// out = (sum over the k ranges, in their order) * scale + bias: the second half of a split
// launch.  VEC consecutive channels per thread.
template <typename XT, int VEC>
__global__ void __launch_bounds__(256) wo_splitk_reduce_kernel(const WoParams p, int splits) {
  const int nv = p.N / VEC;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)p.M * nv) return;
  const int m = (int)(idx / nv), n = (int)(idx % nv) * VEC;
  const int64_t plane = (int64_t)p.M * p.N;
  const float* src = p.partial + (int64_t)m * p.N + n;
  float sum[VEC];
  if constexpr (VEC == 4) {
    f4 v = *reinterpret_cast<const f4*>(src);
    for (int s = 1; s < splits; ++s) v += *reinterpret_cast<const f4*>(src + s * plane);
    sum[0] = v.x, sum[1] = v.y, sum[2] = v.z, sum[3] = v.w;
  } else {
    sum[0] = src[0];
    for (int s = 1; s < splits; ++s) sum[0] += src[s * plane];
  }
  const XT* scale = static_cast<const XT*>(p.scale);
  const XT* bias = static_cast<const XT*>(p.bias);
  XT* out = static_cast<XT*>(p.out) + (int64_t)m * p.ldo + n;
#pragma unroll
  for (int e = 0; e < VEC; ++e)
    out[e] = (XT)(sum[e] * to_f32(scale[n + e]) + (bias ? to_f32(bias[n + e]) : 0.0f));
}

// ---------------------------------------------------------------- small-M kernel, M <= 32 MT
// MT blocks of 32 rows against 32 output channels per workgroup: the weights of those
// channels are read once, whatever M.
template <typename XT, int NW, int MT>
__global__ void __launch_bounds__(NW * 64) wo_skinny_kernel(const WoParams p) {
  __shared__ float red[NW - 1][16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int n = min(n0 + r, p.N - 1);
  const XT* xrow[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
    xrow[i] = static_cast<const XT*>(p.x) + (int64_t)min(i * 32 + r, p.M - 1) * p.ldx + 16 * g;
  const uint8_t* wrow = p.w + (int64_t)n * p.w_sn + 16 * g;
  const h2 c = centre(p, n);
  f16v acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
  const u4 zero = {0, 0, 0, 0};
  // chunks of 32 dealt round-robin over the waves, U in flight per wave: with one byte per
  // weight from HBM the kernel lives on the bytes it keeps in flight
  constexpr int U = MT == 1 ? 4 : (MT == 4 && sizeof(XT) == 4 ? 1 : 2);   // (register budget)
  for (int k0 = wave * 32; k0 < p.K; k0 += U * NW * 32) {
    XFrag<XT> xf[U][MT];
    u4 wf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + u * NW * 32;
      const bool valid = kk + 16 * g < p.K;
      const int k = valid ? kk : 0;
      wf[u] = valid ? *reinterpret_cast<const u4*>(wrow + k) : zero;
#pragma unroll
      for (int i = 0; i < MT; ++i) xf[u][i].load(xrow[i] + k, valid);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      h8 w0, w1;
      widen16(wf[u], p.flip, c, w0, w1);
#pragma unroll
      for (int part = 0; part < XFrag<XT>::kParts; ++part)
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[u][i].step(part, 0), w0, acc[i], 0, 0,
                                                          0);
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[u][i].step(part, 1), w1, acc[i], 0, 0,
                                                          0);
        }
    }
  }
  // partial sums of the waves, one row block at a time through the same 28 KiB of LDS
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    if (i > 0) __syncthreads();
    if (wave > 0) {
#pragma unroll
      for (int v = 0; v < 16; ++v) red[wave - 1][v][lane] = acc[i][v];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int w = 1; w < NW; ++w)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] += red[w - 1][v][lane];
      store_frag<XT>(p, acc[i], i * 32, n0 + r, lane);
    }
  }
}

// ---------------------------------------------------------------- M <= 2: matrix times one or two vectors
// One wave per output channel streams that channel's weight row from end to end -- 64 lanes x
// 16 bytes = 1 KiB contiguous per load instruction, U of them in flight -- and multiplies it
// with the activation rows, which the workgroup keeps in LDS (f32 ones as hi and lo halves),
// on the vector ALUs (v_dot2_f32_f16: the matrix cores have nothing to gain on one or two
// rows, and a row read linearly keeps one DRAM page open where 16 rows read side by side keep
// 16).  The lanes' partial sums meet in a butterfly of cross-lane shuffles.
template <typename XT, int NW, int MR, int U>
__global__ void __launch_bounds__(NW * 64) wo_gemv_kernel(const WoParams p) {
  constexpr bool F32 = sizeof(XT) == 4;
  extern __shared__ __attribute__((aligned(16))) uint8_t wo_lds[];   // [MR][hi | lo][K] halves
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * NW + __builtin_amdgcn_readfirstlane(wave);
  const int kpad = (p.K + 7) & ~7;                       // (K % 16 == 0 anyway)
  // the activation rows into LDS, 8 elements per thread and step
  for (int i = threadIdx.x; i < MR * (kpad >> 3); i += NW * 64) {
    const int m = i / (kpad >> 3), k = (i - m * (kpad >> 3)) << 3;
    const XT* src = static_cast<const XT*>(p.x) + (int64_t)min(m, p.M - 1) * p.ldx + k;
    h8 hi, lo;
    if constexpr (F32) {
      const f4 a = *reinterpret_cast<const f4*>(src), b = *reinterpret_cast<const f4*>(src + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float v = e < 4 ? a[e] : b[e - 4];
        hi[e] = (_Float16)v;
        lo[e] = (_Float16)(v - (float)hi[e]);
      }
      *reinterpret_cast<h8*>(&wo_lds[((2 * m + 1) * kpad + k) * 2]) = lo;
      *reinterpret_cast<h8*>(&wo_lds[((2 * m) * kpad + k) * 2]) = hi;
    } else {
      *reinterpret_cast<h8*>(&wo_lds[(m * kpad + k) * 2]) = *reinterpret_cast<const h8*>(src);
    }
  }
  __syncthreads();
  if (n >= p.N) return;                                  // (no barrier below)
  const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(p.w + (int64_t)n * p.w_sn), 0, p.K, kBufferWord3);
  const h2 c = centre(p, n);
  float acc[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) acc[m] = 0.0f;
  for (int k0 = 16 * lane; k0 < p.K; k0 += U * 1024) {
    u4 wq[U];
#pragma unroll
    for (int u = 0; u < U; ++u)                          // (past K: zeros, no memory touched)
      wq[u] = __builtin_amdgcn_raw_buffer_load_b128(wrs, k0 + u * 1024, 0, 0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u * 1024;
      if (k < p.K) {
        h8 w0, w1;
        widen16(wq[u], p.flip, c, w0, w1);
#pragma unroll
        for (int m = 0; m < MR; ++m) {
#pragma unroll
          for (int part = 0; part < (F32 ? 2 : 1); ++part) {
            const uint8_t* xs = &wo_lds[(((F32 ? 2 * m + part : m) * kpad) + k) * 2];
            const h8 x0 = *reinterpret_cast<const h8*>(xs), x1 = *reinterpret_cast<const h8*>(xs + 16);
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              acc[m] = __builtin_amdgcn_fdot2((h2){x0[e], x0[e + 1]}, (h2){w0[e], w0[e + 1]}, acc[m], false);
              acc[m] = __builtin_amdgcn_fdot2((h2){x1[e], x1[e + 1]}, (h2){w1[e], w1[e + 1]}, acc[m], false);
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    float v = acc[m];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if (lane == 0 && m < p.M) {
      const float sc = to_f32(static_cast<const XT*>(p.scale)[n]);
      const float b = p.bias ? to_f32(static_cast<const XT*>(p.bias)[n]) : 0.0f;
      static_cast<XT*>(p.out)[(int64_t)m * p.ldo + n] = (XT)(v * sc + b);
    }
  }
}

// ---------------------------------------------------------------- 8 < M <= 32, operands through LDS
// 32 output channels per workgroup like wo_skinny_kernel<.., 1>, the k range dealt over the
// waves in units of 64.  There every lane fetches its own activation row (32 rows x 32 bytes
// per load instruction), and from nine rows on the compute unit's address path, not HBM, sets
// the pace.  Here a wave loads each unit the way memory likes it -- eight lanes (sixteen for
// f32) per 128-byte (256-byte) row segment of the activations, four per 64-byte segment of the
// weights --, keeps three units in registers on their way from memory, and turns them into MFMA
// fragments through a piece of LDS that only this wave touches (no barrier: the LDS executes a
// wave's instructions in order).  f32 activations are split into hi and lo half tiles there.
// MR: rows staged (16 or 32).
template <typename XT, int NW, int MR>
__global__ void __launch_bounds__(NW * 64) wo_skinny_lds_kernel(const WoParams p) {
  constexpr bool F32 = sizeof(XT) == 4;
  constexpr int XL = F32 ? 16 : 8;                       // lanes per activation row of a unit
  constexpr int XP = MR * XL / 64;                       // activation loads per lane and unit
  constexpr int XBYTES = MR * 128 * (F32 ? 2 : 1);       // [hi, then lo] half tiles
  constexpr int WBYTES = 32 * 64;
  constexpr int D = 3;                                   // units in registers
  static_assert(D * (XP + 2) <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(16))) uint8_t wo_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int nrows = min(32, p.N - n0), mrows = min(MR, p.M);
  uint8_t* const xs = wo_lds + wave * (XBYTES + WBYTES);
  uint8_t* const ws = xs + XBYTES;
  // descriptors over the activation rows and this workgroup's weight rows; the host has
  // checked that the byte offsets fit 31 bits
  const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void*>(p.x), 0, (int)(((int64_t)(mrows - 1) * p.ldx + p.K) * sizeof(XT)),
      kBufferWord3);
  const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(p.w + (int64_t)n0 * p.w_sn), 0,
      (int)((int64_t)(nrows - 1) * p.w_sn + p.K), kBufferWord3);
  constexpr int kPast = (int)0x80000000;                 // an offset no descriptor covers

  // global -> LDS assignment
  const int xc = lane & (XL - 1), wc = lane & 3;
  int xo[XP], xl[XP];
  bool xok[XP];
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const int row = lane / XL + (64 / XL) * i;
    const int sx = (row ^ (row >> 3)) & 7;
    xok[i] = row < mrows;                                // (rows past M are never stored)
    xo[i] = (int)((int64_t)min(row, mrows - 1) * p.ldx * sizeof(XT)) + 16 * xc;
    xl[i] = F32 ? row * 128 + (((xc >> 1) ^ sx) << 4) + 8 * (xc & 1)
                : row * 128 + ((xc ^ sx) << 4);
  }
  int wo[2], wl[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = (lane >> 2) + 16 * i;
    wo[i] = (int)((int64_t)min(row, nrows - 1) * p.w_sn) + 16 * wc;
    wl[i] = row * 64 + ((wc ^ ((row >> 2) & 3)) << 4);
  }
  const h2 c = centre(p, n0 + min(r, nrows - 1));
  u4 xr[D][XP], wr[D][2];
  auto fetch = [&](u4* xq, u4* wq, int k0) {
    const bool xv = k0 + (F32 ? 4 : 8) * xc < p.K, wv = k0 + 16 * wc < p.K;   // K % 16 == 0
#pragma unroll
    for (int i = 0; i < XP; ++i)
      xq[i] = __builtin_amdgcn_raw_buffer_load_b128(
          xrs, xv && xok[i] ? xo[i] + (int)sizeof(XT) * k0 : kPast, 0, 0);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      wq[i] = __builtin_amdgcn_raw_buffer_load_b128(wrs, wv ? wo[i] + k0 : kPast, 0, 0);
  };
  auto park = [&](const u4* xq, const u4* wq) {
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      if constexpr (F32) {
        const f4 v = __builtin_bit_cast(f4, xq[i]);
        h4 hi, lo;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          hi[e] = (_Float16)v[e];
          lo[e] = (_Float16)(v[e] - (float)hi[e]);
        }
        *reinterpret_cast<h4*>(&xs[xl[i]]) = hi;
        *reinterpret_cast<h4*>(&xs[MR * 128 + xl[i]]) = lo;
      } else {
        *reinterpret_cast<u4*>(&xs[xl[i]]) = xq[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<u4*>(&ws[wl[i]]) = wq[i];
  };
  f16v acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  // this lane's fragment rows (activation rows past the staged ones re-read a staged one:
  // their results are not stored)
  const int xrow = r & (MR - 1), sxr = (xrow ^ (xrow >> 3)) & 7, swr = (r >> 2) & 3;
  auto multiply = [&]() {
#pragma unroll
    for (int q = 0; q < 2; ++q) {                          // the unit's two 32-deep chunks
      const int cx = 4 * q + 2 * g;
      const h8 a0 = *reinterpret_cast<const h8*>(&xs[xrow * 128 + ((cx ^ sxr) << 4)]);
      const h8 a1 = *reinterpret_cast<const h8*>(&xs[xrow * 128 + (((cx + 1) ^ sxr) << 4)]);
      const u4 wq = *reinterpret_cast<const u4*>(&ws[r * 64 + (((2 * q + g) ^ swr) << 4)]);
      h8 w0, w1;
      widen16(wq, p.flip, c, w0, w1);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, w0, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, w1, acc, 0, 0, 0);
      if constexpr (F32) {
        const h8 l0 =
            *reinterpret_cast<const h8*>(&xs[MR * 128 + xrow * 128 + ((cx ^ sxr) << 4)]);
        const h8 l1 =
            *reinterpret_cast<const h8*>(&xs[MR * 128 + xrow * 128 + (((cx + 1) ^ sxr) << 4)]);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(l0, w0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(l1, w1, acc, 0, 0, 0);
      }
    }
  };
  // units wave, wave + NW, ... of 64 of k; set u holds unit i + u on its way from memory
  // (past K: zeros, no memory touched).  The scheduling barriers keep a later step's arithmetic
  // on loaded registers from being moved up to where it would wait for their loads.
  const int w64 = __builtin_amdgcn_readfirstlane(wave) * 64;
#pragma unroll
  for (int d = 0; d < D; ++d) fetch(xr[d], wr[d], w64 + d * NW * 64);
  __builtin_amdgcn_sched_barrier(0);
  for (int k0 = w64; k0 < p.K; k0 += D * NW * 64) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      park(xr[u], wr[u]);
      fetch(xr[u], wr[u], k0 + (D + u) * NW * 64);
      multiply();
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // partial sums of the waves through LDS (all waves are done with their pieces of it)
  __syncthreads();
  float* const red = reinterpret_cast<float*>(wo_lds);   // [NW - 1][16][64]
  if (wave > 0) {
#pragma unroll
    for (int v = 0; v < 16; ++v) red[((wave - 1) * 16 + v) * 64 + lane] = acc[v];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < NW; ++w)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] += red[((w - 1) * 16 + v) * 64 + lane];
    store_frag<XT>(p, acc, 0, n0 + r, lane);
  }
}

// ---------------------------------------------------------------- M <= 16
// 16 output channels per workgroup on v_mfma_f32_16x16x32_f16: twice as many workgroups as the
// 32-channel form for the same weights (a 4096 x 4096 weight gives 256 instead of 128), and a
// lane (row, g) takes the 16 consecutive k values k0 + 16 g .. of a 64-deep chunk, so a wave's
// load covers 64 contiguous bytes of each of its 16 weight rows.
typedef float f4v __attribute__((ext_vector_type(4)));

template <typename XT, int NW>
__global__ void __launch_bounds__(NW * 64) wo_skinny16_kernel(const WoParams p) {
  __shared__ float red[NW - 1][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int n = min(n0 + r, p.N - 1);
  const XT* xrow = static_cast<const XT*>(p.x) + (int64_t)min(r, p.M - 1) * p.ldx + 16 * g;
  const uint8_t* wrow = p.w + (int64_t)n * p.w_sn + 16 * g;
  const h2 c = centre(p, n);
  f4v acc = {0.f, 0.f, 0.f, 0.f};
  const u4 zero = {0, 0, 0, 0};
  constexpr int U = 4;
  for (int k0 = wave * 64; k0 < p.K; k0 += U * NW * 64) {
    XFrag<XT> xf[U];
    u4 wf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + u * NW * 64;
      const bool valid = kk + 16 * g < p.K;              // K % 16 == 0: whole 16-chunks
      const int k = valid ? kk : 0;
      wf[u] = valid ? *reinterpret_cast<const u4*>(wrow + k) : zero;
      xf[u].load(xrow + k, valid);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      h8 w0, w1;
      widen16(wf[u], p.flip, c, w0, w1);
#pragma unroll
      for (int part = 0; part < XFrag<XT>::kParts; ++part) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[u].step(part, 0), w0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[u].step(part, 1), w1, acc, 0, 0, 0);
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave - 1][v][lane] = acc[v];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < NW; ++w)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[v] += red[w - 1][v][lane];
    // D of the 16x16 MFMA: column n = lane % 16, rows 4 (lane / 16) + v
    const int nn = n0 + r;
    if (nn < p.N) {
      const float s = to_f32(static_cast<const XT*>(p.scale)[nn]);
      const float b = p.bias ? to_f32(static_cast<const XT*>(p.bias)[nn]) : 0.0f;
      XT* out = static_cast<XT*>(p.out);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = 4 * g + v;
        if (m < p.M) out[(int64_t)m * p.ldo + nn] = (XT)(acc[v] * s + b);
      }
    }
  }
}

// ---------------------------------------------------------------- any layout, any alignment
template <typename XT>
__global__ void __launch_bounds__(256) wo_generic_kernel(const WoParams p) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)p.M * p.N) return;
  const int m = (int)(idx / p.N), n = (int)(idx % p.N);
  const XT* x = static_cast<const XT*>(p.x) + (int64_t)m * p.ldx;
  const uint8_t* w = p.w + (int64_t)n * p.w_sn;
  const int zp = p.zp ? p.zp[n] : 0;
  float acc = 0.0f;
  for (int k = 0; k < p.K; ++k) {
    const uint8_t b = w[(int64_t)k * p.w_sk];
    const int q = p.flip ? (int)(int8_t)b : (int)b;
    acc += to_f32(x[k]) * (float)(q - zp);
  }
  const float s = to_f32(static_cast<const XT*>(p.scale)[n]);
  const float b = p.bias ? to_f32(static_cast<const XT*>(p.bias)[n]) : 0.0f;
  static_cast<XT*>(p.out)[(int64_t)m * p.ldo + n] = (XT)(acc * s + b);
}

template <typename XT, int WM, int FM, int FN, int SETS>
int launch_lds(dim3 grid, const WoParams& p, hipStream_t st) {
  constexpr int lds = 2 * (WM * FM * 32 * (int)(sizeof(XT) / 2) + 2 * FN * 32) * 128;
  static_assert(lds <= 160 * 1024, "the stages fit the LDS");
  auto kern = wo_lds_kernel<XT, WM, FM, FN, SETS>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (lds > 64 * 1024)
    if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds, &lds_allowed)) return s;
  hipLaunchKernelGGL(kern, grid, dim3(WM * 128), lds, st, p);
  return check_hip(hipGetLastError(), "dq8_weight_only_qgemm launch");
}

template <typename XT, int MR, int U>
int launch_gemv(const WoParams& p, hipStream_t st) {
  const int lds = MR * ((p.K + 7) & ~7) * (int)sizeof(XT);
  auto kern = wo_gemv_kernel<XT, 8, MR, U>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, &lds_allowed)) return s;
  hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(p.N, 8)), dim3(512), lds, st, p);
  return check_hip(hipGetLastError(), "dq8_weight_only_qgemm launch");
}

template <typename XT, int MR>
int launch_skinny_lds(const WoParams& p, hipStream_t st) {
  constexpr int lds = 8 * (MR * 128 * (int)(sizeof(XT) / 2) + 32 * 64);
  static_assert(lds >= 7 * 16 * 64 * 4, "the partial sums of the waves fit");
  auto kern = wo_skinny_lds_kernel<XT, 8, MR>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (lds > 64 * 1024)
    if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds, &lds_allowed)) return s;
  hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(p.N, 32)), dim3(512), lds, st, p);
  return check_hip(hipGetLastError(), "dq8_weight_only_qgemm launch");
}

// The small tile forms of the LDS kernel, for problems whose tiles would leave most of the chip
// idle.  A lone workgroup on a compute unit runs its k tiles as a chain of latencies (LDS
// reads, MFMAs, hand-over of the next tile, barrier): 0.4 us per k tile with two 32 x 32
// fragments per wave, 0.27 us with one -- so below a few rounds of tiles the 64 x 64 tile on
// four waves beats every larger one, although it moves the most bytes per MFMA.
enum { kForm64x64w2 = 0, kForm128x64, kForm64x128w2, kForm128x128, kForm64x64, kNumForms };
struct TileForm { int bm, bn; };
constexpr TileForm kForms[kNumForms] = {{64, 64}, {128, 64}, {64, 128}, {128, 128}, {64, 64}};

// Plan: `splits` workgroups per tile of form `form`, each over k_split of the k range, and
// (splits > 1) a reduction kernel behind them.  `us`: the estimate it was chosen by.
struct SplitPlan {
  int form;
  int splits;
  int k_split;
  float us;
};

// Estimated time of a plan in microseconds, fitted (least squares on relative error, median
// error 4 %, 90th percentile 10 %) to 3300 timed launches of the 64 x 64 and 128 x 128 forms:
// M = 40 .. 3072, nine weight shapes from 768 x 768 to 8192 x 8192, 1 .. 16 k ranges.
//   t = c0 + kt (c1 + c2 (r - 1)) + c3 (r - 1) + [splits > 1] (c4 + c5 M N splits / 1e6)
// kt: 64-deep k tiles per workgroup; r: workgroups per compute unit, rounded up.
struct FormCost { float c0, c1, c2, c3, c4, c5; };
constexpr FormCost kCost64x64[2] = {{4.272f, 0.274f, 0.177f, 0.472f, 2.347f, 1.649f},     // f16
                                    {5.805f, 0.456f, 0.334f, 0.613f, 1.023f, 1.731f}};    // f32
constexpr FormCost kCost128x128[2] = {{7.616f, 0.569f, 0.484f, -0.948f, 1.629f, 1.696f},
                                      {8.471f, 0.919f, 1.175f, -1.589f, -1.035f, 2.310f}};

// The cheapest of the 64 x 64 and 128 x 128 forms with 1, 2, 3, 4, 6 or 8 k ranges of at
// least 192 (one range only unless `may_split`).  Choosing by this estimate comes within
// 1.2 % (geometric mean; worst case 14 %) of the best timed plan of each of those problems.
SplitPlan plan_split(int64_t M, int64_t N, int64_t K, int esz, bool may_split = true) {
  SplitPlan best = {kForm128x128, 1, (int)K, 0.0f};
  const int64_t cus = compute_units();
  for (int form : {(int)kForm64x64, (int)kForm128x128}) {
    const FormCost& c = (form == kForm64x64 ? kCost64x64 : kCost128x128)[esz == 4];
    const int64_t tiles = ceil_div(M, kForms[form].bm) * ceil_div(N, kForms[form].bn);
    for (int want : {1, 2, 3, 4, 6, 8}) {
      if (want > 1 && (!may_split || K / want < 192)) break;
      const int64_t k_split = ceil_div(ceil_div(K, (int64_t)want), 64) * 64;
      const int64_t splits = ceil_div(K, k_split);
      const float kt = (float)(k_split / 64), r = (float)(ceil_div(tiles * splits, cus) - 1);
      float us = c.c0 + kt * (c.c1 + c.c2 * r) + c.c3 * r;
      if (splits > 1) us += c.c4 + c.c5 * (float)((double)M * (double)N * (double)splits * 1e-6);
      if (best.us == 0.0f || us < best.us)
        best = {form, (int)splits, splits > 1 ? (int)k_split : (int)K, us};
    }
  }
  return best;
}

// The 256-row tiles of f16 activations (eight waves, wave tiles 64 x 64 and 64 x 128: the
// larger the wave tile, the fewer LDS bytes per MFMA) against 128 x 128 ones, by the measured
// time of a round of each at 4096 of k: 128 x 128 tiles, two workgroups to a compute unit,
// 82 us for a full round and 45 while one workgroup has the unit to itself; 256 x 128 tiles,
// one to a unit, 75 us and 60 up to half a round; 256 x 256 tiles 135 us and 100.
struct BigTiles {
  int64_t n256x128, n256;     // tiles of the two shapes
  int64_t cost128, cost256x128, cost256;
  bool take256() const { return cost256 < cost128 && cost256 <= cost256x128; }
  bool take256x128() const { return !take256() && cost256x128 < cost128; }
};
BigTiles big_tiles(int64_t M, int64_t N) {
  const int64_t cus = compute_units();
  auto rounds = [](int64_t tiles, int64_t slots, int64_t half, int full_us, int part_us) {
    const int64_t rem = tiles % slots;
    return tiles / slots * full_us + (rem == 0 ? 0 : rem <= half ? part_us : full_us);
  };
  BigTiles b;
  b.n256x128 = ceil_div(M, 256) * ceil_div(N, 128);
  b.n256 = ceil_div(M, 256) * ceil_div(N, 256);
  b.cost128 = rounds(ceil_div(M, 128) * ceil_div(N, 128), 2 * cus, cus, 82, 45);
  b.cost256x128 = rounds(b.n256x128, cus, cus / 2, 75, 60);
  b.cost256 = rounds(b.n256, cus, cus / 2, 135, 100);
  return b;
}

// Estimated time of whichever 256-row tile big_tiles prefers to 128 x 128: 8 us + 0.85 x its
// rounds scaled to K (fitted to 70 timed launches, median error 9 %); 0 where it prefers none.
float big_tile_us(int64_t M, int64_t N, int64_t K) {
  const BigTiles b = big_tiles(M, N);
  const int64_t cost = b.take256() ? b.cost256 : b.take256x128() ? b.cost256x128 : 0;
  return cost ? 8.0f + 0.85f * (float)cost * (float)K / 4096.0f : 0.0f;
}

// The plan for M x N x K, or form = -1 where the small forms are not the choice: up to 32
// rows (16 for f32 activations from 2048 of k on, where the staged kernel pays for two half
// tiles: M = 32, 4096 -> 11008: 25.5 against 33.5 us; 4096^2: 15.7 against 17.9; 8192^2: 33.1
// against 31.2) the kernels for few rows, and the 256-row tiles where they are estimated
// cheaper.
SplitPlan choose_small(int64_t M, int64_t N, int64_t K, int esz, bool may_split) {
  const SplitPlan none = {-1, 1, (int)K, 0.0f};
  // (f32, between: 1536 x 1536 weights, M = 24: 10.0 against 11.2 us, M = 17: 9.5 against 9.2;
  // 768 -> 3072, M = 24: 8.7 against 7.6)
  if (M <= (esz == 4 && K >= 2048 ? 16 : esz == 4 && K >= 1280 ? 23 : 32)) return none;
  const SplitPlan s = plan_split(M, N, K, esz, may_split);
  if (esz == 2 && M > 128) {
    const float big = big_tile_us(M, N, K);
    if (big > 0.0f && big < s.us) return none;
  }
  return s;
}

size_t split_bytes(const SplitPlan& s, int64_t M, int64_t N) {
  return s.splits > 1 ? (size_t)s.splits * (size_t)(M * N) * sizeof(float) : 0;
}

// one launch of a small tile form over the whole k range (splits == 1) or its split
template <typename XT>
int launch_form(int form, int splits, const WoParams& p, hipStream_t st) {
  constexpr int kSets = sizeof(XT) == 2 ? 4 : 2;         // (f32 rows are twice the registers)
  const dim3 grid((unsigned)(ceil_div(p.M, kForms[form].bm) * ceil_div(p.N, kForms[form].bn)),
                  (unsigned)splits);
  switch (form) {
    case kForm64x64w2: return launch_lds<XT, 1, 2, 1, kSets>(grid, p, st);
    case kForm128x64: return launch_lds<XT, 2, 2, 1, kSets>(grid, p, st);
    case kForm64x128w2: return launch_lds<XT, 1, 2, 2, kSets>(grid, p, st);
    case kForm128x128:
      if constexpr (sizeof(XT) == 4) return launch_lds<XT, 4, 1, 2, kSets>(grid, p, st);
      return launch_lds<XT, 2, 2, 2, kSets>(grid, p, st);
    case kForm64x64: return launch_lds<XT, 2, 1, 1, kSets>(grid, p, st);
  }
  return fail("dq8_weight_only_qgemm: unknown tile form");
}

template <typename XT>
int launch(WoParams& p, bool fast, void* scratch, size_t scratch_bytes, hipStream_t st) {
  p.partial = nullptr;
  p.k_split = p.K;
  // (the LDS kernel addresses a tile's rows by 31-bit byte offsets from its first)
  const bool lds_ok = 512 * p.ldx + 4 * (int64_t)p.K + 4096 < (1LL << 31) &&
                      256 * p.w_sn + (int64_t)p.K + 4096 < (1LL << 31);
  if (fast && lds_ok) {
    const bool have = scratch && aligned(scratch, 16);
    SplitPlan s = choose_small(p.M, p.N, p.K, (int)sizeof(XT), have);
    if (s.splits > 1 && scratch_bytes < split_bytes(s, p.M, p.N))
      s = choose_small(p.M, p.N, p.K, (int)sizeof(XT), false);
    if (s.form >= 0 && s.splits > 1) {
      const int sp = s.splits;
      p.partial = static_cast<float*>(scratch);
      p.k_split = s.k_split;
      if (int e = launch_form<XT>(s.form, sp, p, st)) return e;
      const int vec = (p.N % 4 == 0 && aligned(p.out, 8) && p.ldo % 4 == 0) ? 4 : 1;
      const int64_t blocks = ceil_div((int64_t)p.M * (p.N / vec), 256);
      DQ8_REQUIRE(blocks < (1LL << 31), "dq8_weight_only_qgemm: problem too large");
      if (vec == 4)
        hipLaunchKernelGGL((wo_splitk_reduce_kernel<XT, 4>), dim3((unsigned)blocks), dim3(256), 0,
                           st, p, sp);
      else
        hipLaunchKernelGGL((wo_splitk_reduce_kernel<XT, 1>), dim3((unsigned)blocks), dim3(256), 0,
                           st, p, sp);
      return check_hip(hipGetLastError(), "dq8_weight_only_qgemm reduction launch");
    }
    if (s.form >= 0) return launch_form<XT>(s.form, 1, p, st);
  }
  if (!fast) {
    const int64_t blocks = ceil_div((int64_t)p.M * p.N, 256);
    DQ8_REQUIRE(blocks < (1LL << 31), "dq8_weight_only_qgemm: problem too large");
    hipLaunchKernelGGL(wo_generic_kernel<XT>, dim3((unsigned)blocks), dim3(256), 0, st, p);
  } else if (p.M <= 128) {
    const unsigned grid = (unsigned)ceil_div(p.N, 32);
    // (with more than 8 rows every workgroup re-reads the activations, which then outweigh
    // its weights: the narrow form only while the wide one would leave compute units idle)
    // (the staged kernel addresses activation and weight rows by 31-bit byte offsets)
    const bool staged_ok =
        ((int64_t)(p.M - 1) * p.ldx + p.K) * (int64_t)sizeof(XT) + 65536 < (1LL << 31) &&
        32 * p.w_sn + (int64_t)p.K + 65536 < (1LL << 31);
    // (it needs several 64-deep units per wave to run its pipeline: measured against the two
    // kernels below it wins from 12 rows on at 3072 and 4096 of k -- 4096^2 weights, f16, M = 32:
    // 10.7 against 14.9 us -- and from 5 rows on at 8192 -- M = 16: 16.8 against 22.5 us --, and
    // loses about a microsecond at 768 or 1040 of k)
    // one row, or two where it was measured faster (f32 activations; f16 from 2048 to 8192 of
    // k), while the rows fit 64 KiB of LDS: the row-streaming kernel on the vector ALUs (4096^2
    // weights, M = 1: f16 4.3 against 5.8 us, f32 4.5 against 7.5; 8192^2: 13.5 against 15.2 us,
    // 5.0 TB/s; three and four rows are slower that way than on the matrix cores)
    if ((p.M == 1 || (p.M == 2 && (sizeof(XT) == 4 || (p.K >= 2048 && p.K <= 8192)))) &&
        (int64_t)p.M * p.K * (int64_t)sizeof(XT) <= 64 * 1024) {
      const bool deep = p.K > 4096;
      if (p.M == 1) return deep ? launch_gemv<XT, 1, 8>(p, st) : launch_gemv<XT, 1, 4>(p, st);
      return deep ? launch_gemv<XT, 2, 8>(p, st) : launch_gemv<XT, 2, 4>(p, st);
    }
    // (and from 5 rows on against weights of at least 8192 channels, where its 32-channel
    // workgroups fill the chip: 4096 -> 16384, M = 8: f16 17.7 against 19.6 us, f32 23.7
    // against 30.5)
    // (three and four rows that way only against narrow weights, where a workgroup per 16
    // channels leaves most compute units idle: 3072 -> 768, M = 4: f16 5.3 against 5.5 us, f32
    // 6.1 against 7.8; 8192 -> 1024: 8.0 against 9.5 and 10.2 against 13.0; at 4096 channels
    // and more the matrix cores win)
    if (p.M >= 3 && p.M <= 4 && p.N <= 1024 && p.K >= 2048 &&
        (int64_t)4 * p.K * (int64_t)sizeof(XT) <= 128 * 1024)
      return p.K > 4096 ? launch_gemv<XT, 4, 8>(p, st) : launch_gemv<XT, 4, 4>(p, st);
    if (staged_ok && p.M <= 32 &&
        ((p.K >= 2048 && p.M >= 12) || (p.M >= 5 && (p.K >= 6144 || (p.K >= 2048 && p.N >= 8192)))))
      return p.M <= 16 ? launch_skinny_lds<XT, 16>(p, st) : launch_skinny_lds<XT, 32>(p, st);
    if (p.M <= 8 || (p.M <= 16 && grid < 256))
      hipLaunchKernelGGL((wo_skinny16_kernel<XT, 8>), dim3((unsigned)ceil_div(p.N, 16)), dim3(512),
                         0, st, p);
    else if (p.M <= 32)
      hipLaunchKernelGGL((wo_skinny_kernel<XT, 8, 1>), dim3(grid), dim3(512), 0, st, p);
    else if (p.M <= 64)
      hipLaunchKernelGGL((wo_skinny_kernel<XT, 8, 2>), dim3(grid), dim3(512), 0, st, p);
    else
      hipLaunchKernelGGL((wo_skinny_kernel<XT, 8, 4>), dim3(grid), dim3(512), 0, st, p);
  } else {
    // (here: the plan above preferred a 256-row tile, or the LDS kernel cannot address the
    // operands and the register kernel takes the problem)
    if constexpr (sizeof(XT) == 2) {
      const BigTiles b = big_tiles(p.M, p.N);
      if (b.take256() && lds_ok)
        return launch_lds<XT, 4, 2, 4, 2>(dim3((unsigned)b.n256), p, st);
      if (b.take256x128() && lds_ok)
        return launch_lds<XT, 4, 2, 2, 4>(dim3((unsigned)b.n256x128), p, st);
    }
    const int64_t big = ceil_div(p.M, 128) * ceil_div(p.N, 128);
    if (big >= 192) {
      hipLaunchKernelGGL((wo_tile_kernel<XT, 2, 2>), dim3((unsigned)big), dim3(256), 0, st, p);
    } else {
      const int64_t small = ceil_div(p.M, 64) * ceil_div(p.N, 64);
      hipLaunchKernelGGL((wo_tile_kernel<XT, 1, 1>), dim3((unsigned)small), dim3(256), 0, st, p);
    }
  }
  return check_hip(hipGetLastError(), "dq8_weight_only_qgemm launch");
}

}  // namespace
}  // namespace dq8

using namespace dq8;

namespace {
// bytes of the [N, K] copy of weights given as [K, N], kept 256-byte aligned
size_t transposed_bytes(int64_t N, int64_t K, int tp_b) {
  return (tp_b || N <= 0 || K <= 0) ? 0 : ((size_t)(N * K) + 255) / 256 * 256;
}
// Undoes the byte permutation the reference's compiler applies to a constant [K, N] ui8 weight
// (R tao_compiler/mlir/disc/transforms/disc_transform_weight_data_layout_for_weight_only_gemm.cc
// :54-300 as composed at :362-370: rows permuted in blocks of 16, transpose, column pairs
// interleaved in tiles of 64 rows, bytes 1 and 2 of every word swapped).  Composed, the 16
// bytes W^T[n, 16 j .. 16 j + 15] sit in one 16-byte group of the reordered buffer, at byte
//   (n / 2) * 2 K + (16 j / 64) * 128 + (n % 2) * 64 + (16 j) % 64,
// even bytes of the group = the first eight k, odd bytes = the last eight.  One thread per
// group: a 16-byte load, four byte permutes, a 16-byte store into the kernels' [N, K] layout.
__global__ void __launch_bounds__(256)
wo_undo_compiler_layout_kernel(const u4* __restrict__ src, u4* __restrict__ dst, int N, int K16) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= (int64_t)N * K16) return;
  const int n = (int)(g / K16), j = (int)(g % K16);
  const int64_t off16 = (int64_t)(n >> 1) * (2 * K16) + (j >> 2) * 8 + (n & 1) * 4 + (j & 3);
  const u4 v = __builtin_nontemporal_load(src + off16);
  u4 r;
  // v_perm_b32 selector bytes: 0-3 pick from the second operand, 4-7 from the first
  r.x = __builtin_amdgcn_perm(v.y, v.x, 0x06040200u);   // k 0..3  = bytes 0,2 of words 0,1
  r.y = __builtin_amdgcn_perm(v.w, v.z, 0x06040200u);   // k 4..7  = bytes 0,2 of words 2,3
  r.z = __builtin_amdgcn_perm(v.y, v.x, 0x07050301u);   // k 8..11 = bytes 1,3 of words 0,1
  r.w = __builtin_amdgcn_perm(v.w, v.z, 0x07050301u);   // k 12..15
  dst[g] = r;
}

}  // namespace

extern "C" size_t dq8_weight_only_qgemm_workspace_bytes(int64_t N, int64_t K, int tp_b) {
  return (tp_b || N <= 0 || K <= 0) ? 0 : (size_t)(N * K);
}

extern "C" size_t dq8_weight_only_qgemm_workspace_bytes_ex(int64_t M, int64_t N, int64_t K,
                                                           int tp_b, int x_dtype) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  size_t split = 0;
  if ((x_dtype == DQ8_DTYPE_F16 || x_dtype == DQ8_DTYPE_F32) && K % 16 == 0 && M < (1LL << 31) &&
      N < (1LL << 31) && K < (1LL << 31))
    split = split_bytes(choose_small(M, N, K, x_dtype == DQ8_DTYPE_F32 ? 4 : 2, true), M, N);
  if (!split) return dq8_weight_only_qgemm_workspace_bytes(N, K, tp_b);
  return transposed_bytes(N, K, tp_b) + split;
}

extern "C" int dq8_weight_only_undo_compiler_layout(const uint8_t* reordered, uint8_t* w_nk,
                                                    int64_t K, int64_t N, void* stream) {
  clear_error();
  DQ8_REQUIRE(K >= 0 && N >= 0 && K < (1LL << 31) && N < (1LL << 31),
              "dq8_weight_only_undo_compiler_layout: bad shape");
  // (outside these shapes the compiler's pass reads and writes out of bounds: not a permutation)
  DQ8_REQUIRE(K % 64 == 0 && N % 4 == 0,
              "dq8_weight_only_undo_compiler_layout: the compiler's weight layout is defined for "
              "K % 64 == 0 and N % 4 == 0 only");
  if (K == 0 || N == 0) return 0;
  DQ8_REQUIRE(reordered && w_nk, "dq8_weight_only_undo_compiler_layout: null pointer");
  DQ8_REQUIRE(aligned(reordered, 16) && aligned(w_nk, 16),
              "dq8_weight_only_undo_compiler_layout: buffers must be 16-byte aligned");
  DQ8_REQUIRE(reordered != w_nk, "dq8_weight_only_undo_compiler_layout: not in place");
  const int64_t groups = N * (K / 16);
  hipLaunchKernelGGL(wo_undo_compiler_layout_kernel, dim3((unsigned)ceil_div(groups, 256)),
                     dim3(256), 0, (hipStream_t)stream, reinterpret_cast<const u4*>(reordered),
                     reinterpret_cast<u4*>(w_nk), (int)N, (int)(K / 16));
  return check_hip(hipGetLastError(), "dq8_weight_only_undo_compiler_layout launch");
}

extern "C" int dq8_weight_only_qgemm(const void* x, int x_dtype, int64_t ldx, const void* w,
                                     int w_signed, int64_t ldw, int tp_b, const void* scale,
                                     const int32_t* zero_points, const void* bias, void* out,
                                     int64_t ldo, int64_t M, int64_t N, int64_t K,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  DQ8_REQUIRE(x_dtype == DQ8_DTYPE_F32 || x_dtype == DQ8_DTYPE_F16,
              "dq8_weight_only_qgemm: activations must be f32 or f16");
  DQ8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "dq8_weight_only_qgemm: negative size");
  DQ8_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K < (1LL << 31),
              "dq8_weight_only_qgemm: size too large");
  if (M == 0 || N == 0) return 0;
  DQ8_REQUIRE(x && w && scale && out, "dq8_weight_only_qgemm: null pointer");
  DQ8_REQUIRE(ldx >= K && ldo >= N && ldw >= (tp_b ? K : N),
              "dq8_weight_only_qgemm: leading dimension too small");
  hipStream_t st = (hipStream_t)stream;
  const int esz = x_dtype == DQ8_DTYPE_F32 ? 4 : 2;
  WoParams p;
  p.x = x;
  p.w = static_cast<const uint8_t*>(w);
  p.scale = scale;
  p.zp = zero_points;
  p.bias = bias;
  p.out = out;
  p.ldx = ldx;
  p.ldo = ldo;
  p.w_sn = tp_b ? ldw : 1;
  p.w_sk = tp_b ? 1 : ldw;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.flip = w_signed ? 0x80808080u : 0u;
  // the MFMA kernels want k-contiguous 16-byte aligned rows of both operands; weights given
  // as [K, N] are transposed into the caller's scratch first (a runtime does that once per
  // constant weight and passes the result with tp_b = 1 from then on)
  bool fast = K > 0 && K % 16 == 0 && aligned(x, 16) && (ldx * esz) % 16 == 0;
  // what the transposed weights leave of the scratch holds the partial sums of a split launch
  void* rest = workspace;
  size_t rest_bytes = workspace ? workspace_bytes : 0;
  if (fast && !tp_b) {
    if (workspace && aligned(workspace, 16) && workspace_bytes >= (size_t)(N * K)) {
      if (int s = dq8_transpose_s8(static_cast<const int8_t*>(w), ldw,
                                   static_cast<int8_t*>(workspace), K, N, stream))
        return s;
      p.w = static_cast<const uint8_t*>(workspace);
      p.w_sn = K;
      p.w_sk = 1;
      const size_t used = transposed_bytes(N, K, 0);
      rest = used < workspace_bytes ? static_cast<char*>(workspace) + used : nullptr;
      rest_bytes = used < workspace_bytes ? workspace_bytes - used : 0;
    } else {
      fast = false;
    }
  }
  fast = fast && aligned(p.w, 16) && p.w_sn % 16 == 0 && p.w_sk == 1;
  return x_dtype == DQ8_DTYPE_F32 ? launch<float>(p, fast, rest, rest_bytes, st)
                                  : launch<_Float16>(p, fast, rest, rest_bytes, st);
}
