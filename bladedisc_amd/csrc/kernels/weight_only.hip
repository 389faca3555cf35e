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
// Both operands go from global memory straight into registers in MFMA layout: the order of
// the k values inside a fragment is free as long as both operands agree, so lane (row, g) takes
// the 16 consecutive k values k0 + 16 g .. of its row -- 16 weight bytes (one dwordx4), 16
// activations -- and feeds two MFMAs with them.
//  * wo_lds_kernel: f16 activations, 128 x 128 tiles shared through LDS, once there are about a
//    hundred of them (256 x 128 on eight waves once those fill the chip; 0.84-0.90 PFLOP/s at
//    4096^2 .. 8192^2 weights, where the ROCm library's plain f16 GEMM reaches 1.16-1.49);
//  * wo_tile_kernel: 2 x 2 waves, wave tile (32 FM) x (32 FN), operands straight into registers:
//    f32 activations and problems with few tiles;
//  * wo_skinny16_kernel: M <= 16 rows against 16 output channels per workgroup (16x16x32 MFMA);
//  * wo_skinny_kernel: M <= 128 rows against 32 output channels per workgroup, the k range dealt
//    over the waves and the partial sums added through LDS (bound by the weight bytes: 1 byte
//    per weight from HBM);
//  * wo_generic_kernel: one output per thread, any layout and alignment (also weights left as
//    [K, N]).
#include "dq8_common.h"
#include "disc_q8.h"

#pragma clang fp contract(off)

namespace dq8 {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));

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
// (64 WM) x 128 tile, WM x 2 waves (WM = 2 or 4), k tiles of 64 in two LDS stages.  The
// register kernel above makes every lane fetch its own row, 64 cache lines per load instruction, and the compute unit's
// address path caps it at about 15 bytes per clock (0.4 PFLOP/s whatever the shape); here
// eight lanes cover one 128-byte row segment of the activations and four one 64-byte segment of
// the weights, the tile is shared through LDS (16-byte chunks XOR-swizzled by the row so that
// the fragment reads spread over the banks), and the fragments are read back as ds_read_b128.
template <int WM, bool WIDE>
__global__ void __launch_bounds__(WM * 128) wo_lds_kernel(const WoParams p) {
  constexpr int BM = WM * 64, BN = 128, BK = 64;
  constexpr int NT = WM * 128;                           // WM x 2 waves
  constexpr int WP = (BN * 4) / NT;                      // weight chunks per thread: 2 or 1
  __shared__ __attribute__((aligned(16))) uint8_t xs[2][BM * BK * 2];
  // WIDE: the weights are widened to halves once, on their way into LDS (128-byte rows like the
  // activations'), not by every wave that reads them
  __shared__ __attribute__((aligned(16))) uint8_t ws[2][BN * BK * (WIDE ? 2 : 1)];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.N + BN - 1) / BN;
  const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;
  const int r = lane & 31, g = lane >> 5;
  const _Float16* x = static_cast<const _Float16*>(p.x);
  const u4 zero = {0, 0, 0, 0};

  // global -> LDS assignment
  const int xc = tid & 7, wc = tid & 3;                  // 16-byte chunk of the row's k tile
  const _Float16* xg[4];
  int xl[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = (tid >> 3) + (NT / 8) * i;
    xg[i] = x + (int64_t)min(m0 + row, p.M - 1) * p.ldx + 8 * xc;
    xl[i] = row * 128 + ((xc ^ ((row ^ (row >> 3)) & 7)) << 4);
  }
  const uint8_t* wg[WP];
  int wl[WP], wl1[WP];
  h2 cpark[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int row = (tid >> 2) + (NT / 4) * i;
    wg[i] = p.w + (int64_t)min(n0 + row, p.N - 1) * p.w_sn + 16 * wc;
    if (WIDE) {
      const int sw = (row ^ (row >> 3)) & 7;
      wl[i] = row * 128 + (((2 * wc) ^ sw) << 4);
      wl1[i] = row * 128 + (((2 * wc + 1) ^ sw) << 4);
      cpark[i] = centre(p, min(n0 + row, p.N - 1));
    } else {
      wl[i] = row * 64 + ((wc ^ ((row >> 2) & 3)) << 4);
      wl1[i] = 0;
    }
  }
  // three register sets: the loads of k tiles t + 1 .. t + 3 are in flight while tile t is
  // multiplied (with one workgroup on a compute unit nothing else covers the load latency)
  u4 xr[3][4], wr[3][WP];
  auto fetch = [&](u4* xq, u4* wq, int k0) {
    const bool xv = k0 + 8 * xc < p.K, wv = k0 + 16 * wc < p.K;   // K % 16 == 0
#pragma unroll
    for (int i = 0; i < 4; ++i) xq[i] = xv ? *reinterpret_cast<const u4*>(xg[i] + k0) : zero;
#pragma unroll
    for (int i = 0; i < WP; ++i) wq[i] = wv ? *reinterpret_cast<const u4*>(wg[i] + k0) : zero;
  };
  auto park = [&](const u4* xq, const u4* wq, int stage) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u4*>(&xs[stage][xl[i]]) = xq[i];
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      if (WIDE) {
        h8 lo, hi;
        widen16(wq[i], p.flip, cpark[i], lo, hi);
        *reinterpret_cast<h8*>(&ws[stage][wl[i]]) = lo;
        *reinterpret_cast<h8*>(&ws[stage][wl1[i]]) = hi;
      } else {
        *reinterpret_cast<u4*>(&ws[stage][wl[i]]) = wq[i];
      }
    }
  };

  // fragment rows of this wave and the weight centres of its columns
  int xrow[2], wrow[2];
  h2 c[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    xrow[i] = wm * 64 + i * 32 + r;
    wrow[i] = wn * 64 + i * 32 + r;
    c[i] = centre(p, min(n0 + wrow[i], p.N - 1));
  }
  f16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  auto multiply = [&](int st) {
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    h8 a0[2], a1[2], w0[2], w1[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c0 = 4 * s + 2 * g, row = xrow[i];
      const int sx = (row ^ (row >> 3)) & 7;
      a0[i] = *reinterpret_cast<const h8*>(&xs[st][row * 128 + ((c0 ^ sx) << 4)]);
      a1[i] = *reinterpret_cast<const h8*>(&xs[st][row * 128 + (((c0 + 1) ^ sx) << 4)]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = wrow[j];
      if (WIDE) {
        const int c0 = 4 * s + 2 * g, sw = (row ^ (row >> 3)) & 7;
        w0[j] = *reinterpret_cast<const h8*>(&ws[st][row * 128 + ((c0 ^ sw) << 4)]);
        w1[j] = *reinterpret_cast<const h8*>(&ws[st][row * 128 + (((c0 + 1) ^ sw) << 4)]);
      } else {
        const int cw = 2 * s + g;
        const u4 q =
            *reinterpret_cast<const u4*>(&ws[st][row * 64 + ((cw ^ ((row >> 2) & 3)) << 4)]);
        widen16(q, p.flip, c[j], w0[j], w1[j]);
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0[i], w0[j], acc[i][j], 0, 0, 0);
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1[i], w1[j], acc[i][j], 0, 0, 0);
      }
  }
  };
  const int KT = (p.K + BK - 1) / BK;
  fetch(xr[0], wr[0], 0);
  fetch(xr[1], wr[1], BK);
  fetch(xr[2], wr[2], 2 * BK);
  park(xr[0], wr[0], 0);
  __syncthreads();
  for (int t0 = 0; t0 < KT; t0 += 6) {
#pragma unroll
    for (int u = 0; u < 6; ++u) {
      const int t = t0 + u;
      if (t < KT) {                                        // (uniform over the workgroup)
        fetch(xr[u % 3], wr[u % 3], (t + 3) * BK);         // (past K: zeros)
        multiply(u % 2);
        if (t + 1 < KT) park(xr[(u + 1) % 3], wr[(u + 1) % 3], (u + 1) % 2);
        __syncthreads();
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      store_frag<_Float16>(p, acc[i][j], m0 + xrow[i] - r, n0 + wrow[j], lane);
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

template <typename XT>
int launch(const WoParams& p, bool fast, hipStream_t st) {
  if (!fast) {
    const int64_t blocks = ceil_div((int64_t)p.M * p.N, 256);
    DQ8_REQUIRE(blocks < (1LL << 31), "dq8_weight_only_qgemm: problem too large");
    hipLaunchKernelGGL(wo_generic_kernel<XT>, dim3((unsigned)blocks), dim3(256), 0, st, p);
  } else if (p.M <= 128) {
    const unsigned grid = (unsigned)ceil_div(p.N, 32);
    // (with more than 8 rows every workgroup re-reads the activations, which then outweigh
    // its weights: the narrow form only while the wide one would leave compute units idle)
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
    // 128 x 128 tiles through LDS once there are enough of them to put several workgroups on
    // a compute unit (a lone workgroup's chain of load, LDS, widen and MFMA latencies is not
    // covered: 48 tiles of a 3072-deep problem take as long through LDS as 192 small tiles
    // through registers); the register kernel below that and for f32 activations
    const int64_t big = ceil_div(p.M, 128) * ceil_div(p.N, 128);
    const int64_t big256 = ceil_div(p.M, 256) * ceil_div(p.N, 128);
    if (big256 >= 384 && sizeof(XT) == 2) {
      hipLaunchKernelGGL((wo_lds_kernel<4, true>), dim3((unsigned)big256), dim3(512), 0, st, p);
    } else if (big >= 96 && sizeof(XT) == 2) {
      hipLaunchKernelGGL((wo_lds_kernel<2, true>), dim3((unsigned)big), dim3(256), 0, st, p);
    } else if (big >= 192) {
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

extern "C" size_t dq8_weight_only_qgemm_workspace_bytes(int64_t N, int64_t K, int tp_b) {
  return (tp_b || N <= 0 || K <= 0) ? 0 : (size_t)(N * K);
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
  if (fast && !tp_b) {
    if (workspace && aligned(workspace, 16) && workspace_bytes >= (size_t)(N * K)) {
      if (int s = dq8_transpose_s8(static_cast<const int8_t*>(w), ldw,
                                   static_cast<int8_t*>(workspace), K, N, stream))
        return s;
      p.w = static_cast<const uint8_t*>(workspace);
      p.w_sn = K;
      p.w_sk = 1;
    } else {
      fast = false;
    }
  }
  fast = fast && aligned(p.w, 16) && p.w_sn % 16 == 0 && p.w_sk == 1;
  return x_dtype == DQ8_DTYPE_F32 ? launch<float>(p, fast, st) : launch<_Float16>(p, fast, st);
}
