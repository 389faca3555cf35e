// Host launchers of the int8 GEMM / convolution kernels for gfx950, the generic
// (any layout, any alignment, zero points) scalar kernels, and the MFMA layout
// probe.  The tile shape is chosen at run time from the dynamic M.
#include <algorithm>
#include <cstdlib>
#include <cmath>

#include "dq8_common.h"
#include "disc_q8.h"
#include "qgemm_device.h"
#include "qgemm_launch.h"
#include "qconv_direct.h"
#include "qconv_stream.h"

#pragma clang fp contract(off)

namespace dq8 {
namespace {

// ------------------------------------------------------------ generic kernels
struct GenericParams {
  const int8_t* A;
  const int8_t* W;
  int64_t a_sm, a_sk;  // element strides of A along m and k
  int64_t w_sn, w_sk;  // element strides of W along n and k
  int K;
  int zx, zw;
  EpiParams epi;
};

template <int EPI>
__device__ __forceinline__ void store_one(const EpiParams& e, int m, int n, int acc) {
  const ColParams c = col_params<EPI>(e, n);
  const int64_t off = (int64_t)m * e.ldo + n;
  if (EPI == DQ8_EPI_ACC_S32)
    ((int32_t*)e.out)[off] = acc;
  else if (EPI == DQ8_EPI_DEQUANT_F32)
    ((float*)e.out)[off] = finish_f32(e, dequant_one_any(e, c, acc, dequant_so(e)), m, n);
  else
    ((int8_t*)e.out)[off] = (int8_t)finish_s8(e, requant_one<EPI>(e, c, acc), m, n);
}

template <int EPI>
__global__ void __launch_bounds__(256) qgemm_generic_kernel(const GenericParams p) {
  const int64_t total = (int64_t)p.epi.M * p.epi.N;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * 256) {
    const int m = (int)(idx / p.epi.N), n = (int)(idx % p.epi.N);
    const int8_t* a = p.A + (int64_t)m * p.a_sm;
    const int8_t* w = p.W + (int64_t)n * p.w_sn;
    int acc = 0;
    for (int k = 0; k < p.K; ++k)
      acc += ((int)a[(int64_t)k * p.a_sk] - p.zx) * ((int)w[(int64_t)k * p.w_sk] - p.zw);
    store_one<EPI>(p.epi, m, n, acc);
  }
}

struct GenericConvParams {
  const int8_t* in;
  const int8_t* w;
  int64_t i_sb, i_sc, i_sh, i_sw;  // input element strides: batch, channel, h, w
  int64_t w_si, w_so, w_sh, w_sw;  // kernel strides: in ch, out ch, h, w
  int64_t o_sb, o_sc, o_sh, o_sw;  // output strides
  int NB, H, Wd, Ci, Co, Kh, Kw, Ho, Wo;
  int pad_t, pad_l, sh, sw_, dh, dw;
  EpiParams epi;  // M = NB*Ho*Wo, N = Co; ldo unused
};

template <int EPI>
__global__ void __launch_bounds__(256) qconv_generic_kernel(const GenericConvParams p) {
  const int64_t total = (int64_t)p.NB * p.Ho * p.Wo * p.Co;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * 256) {
    const int co = (int)(idx % p.Co);
    int64_t r = idx / p.Co;
    const int x = (int)(r % p.Wo);
    r /= p.Wo;
    const int y = (int)(r % p.Ho);
    const int b = (int)(r / p.Ho);
    int acc = 0;
    for (int kh = 0; kh < p.Kh; ++kh) {
      const int yy = y * p.sh - p.pad_t + kh * p.dh;
      if (yy < 0 || yy >= p.H) continue;
      for (int kw = 0; kw < p.Kw; ++kw) {
        const int xx = x * p.sw_ - p.pad_l + kw * p.dw;
        if (xx < 0 || xx >= p.Wd) continue;
        const int8_t* pi = p.in + b * p.i_sb + yy * p.i_sh + xx * p.i_sw;
        const int8_t* pw = p.w + co * p.w_so + kh * p.w_sh + kw * p.w_sw;
        for (int ci = 0; ci < p.Ci; ++ci)
          acc += (int)pi[ci * p.i_sc] * (int)pw[ci * p.w_si];
      }
    }
    const ColParams c = col_params<EPI>(p.epi, co);
    const int64_t off = b * p.o_sb + co * p.o_sc + y * p.o_sh + x * p.o_sw;
    if (EPI == DQ8_EPI_ACC_S32)
      ((int32_t*)p.epi.out)[off] = acc;
    else if (EPI == DQ8_EPI_DEQUANT_F32)   // (a fused residual has the output's layout)
      ((float*)p.epi.out)[off] = finish_f32_at(p.epi, dequant_one_any(p.epi, c, acc, dequant_so(p.epi)), off);
    else
      ((int8_t*)p.epi.out)[off] = (int8_t)finish_s8_at(p.epi, requant_one<EPI>(p.epi, c, acc), off);
  }
}

// int8 [R, C] (row stride ld) -> [C, R] with row stride ldd >= R, columns R .. ldd-1 zero;
// 64x64 tiles through LDS, blockIdx.y over ceil(ldd / 64)
__global__ void __launch_bounds__(256)
transpose_s8_kernel(const int8_t* __restrict__ src, int64_t ld, int8_t* __restrict__ dst,
                    int R, int C, int ldd) {
  __shared__ int8_t tile[64][65];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    tile[i][tx] = (r < R && c < C) ? src[(int64_t)r * ld + c] : (int8_t)0;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, r = r0 + tx;
    if (c < C && r < ldd) dst[(int64_t)c * ldd + r] = tile[tx][i];   // (zero for r >= R)
  }
}

// dst[b][c][r] = src[b][r][c] for B dense matrices [R, C] of 1- or 4-byte elements (layout
// changes between NCHW and NHWC, OIHW and OHWI); 32x32 tiles through LDS
template <typename T>
__global__ void __launch_bounds__(256)
transpose_batched_kernel(const T* __restrict__ src, T* __restrict__ dst, int R, int C,
                         int tiles_c) {
  __shared__ T tile[32][33];
  const int64_t base = (int64_t)blockIdx.y * R * C;
  const int r0 = (blockIdx.x / tiles_c) * 32, c0 = (blockIdx.x % tiles_c) * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int i = ty; i < 32; i += 8) {
    const int r = r0 + i, c = c0 + tx;
    if (r < R && c < C) tile[i][tx] = src[base + (int64_t)r * C + c];
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    const int c = c0 + i, r = r0 + tx;
    if (c < C && r < R) dst[base + (int64_t)c * R + r] = tile[tx][i];
  }
}

template <typename T>
int transpose_batched(const void* src, void* dst, int64_t B, int64_t R, int64_t C,
                      hipStream_t st) {
  if (B == 0 || R == 0 || C == 0) return 0;
  const int64_t tiles_c = ceil_div(C, 32), tiles = ceil_div(R, 32) * tiles_c;
  DQ8_REQUIRE(B <= 65535 && tiles < (1LL << 31), "layout change: tensor too large");
  hipLaunchKernelGGL(transpose_batched_kernel<T>, dim3((unsigned)tiles, (unsigned)B), dim3(256), 0,
                     st, static_cast<const T*>(src), static_cast<T*>(dst), (int)R, (int)C,
                     (int)tiles_c);
  return check_hip(hipGetLastError(), "layout change launch");
}

// Space to depth for stride-2 convolutions of images with at most 4 channels (the stem of a
// vision network: 7 x 7, stride 2, 3 channels).  src: [B, H, W, C] with C <= 4; the element
// at padded position (2 by + dy, 2 bx + dx), channel c goes to dst[b][by][bx][(2 dy + dx) C + c]
// of [B, Hb, Wb, 16]; positions in the padding frame and the channels past 4 C are zero.  A
// K x K stride-2 convolution of src is then a ceil(K / 2)^2 stride-1 convolution of dst.  With
// H = Kh, W = Kw, no padding and B = Co the same kernel re-lays out the weights.  One 16-byte
// store per thread.
// One launch does two such jobs (image and weights): blockIdx.y < a.B belongs to the first.
struct SpaceToDepthJob {
  const int8_t* src;
  int8_t* dst;
  int B, H, W, Hb, Wb, pad_t, pad_l;
};
template <int C>
__global__ void __launch_bounds__(256)
space_to_depth2_s8_kernel(const SpaceToDepthJob ja, const SpaceToDepthJob jb) {
  // blockIdx.y: image; threads over its Hb * Wb output pixels
  const bool first = (int)blockIdx.y < ja.B;
  const SpaceToDepthJob& j = first ? ja : jb;
  const int8_t* __restrict__ src = j.src;
  int8_t* __restrict__ dst = j.dst;
  const int H = j.H, W = j.W, Hb = j.Hb, Wb = j.Wb, pad_t = j.pad_t, pad_l = j.pad_l;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= Hb * Wb) return;
  const int by = idx / Wb, bx = idx - by * Wb;
  const int64_t b = first ? (int)blockIdx.y : (int)blockIdx.y - ja.B;
  // the two pixels of an image row that go into one output pixel are 2 C consecutive bytes
  // there and here: one (unaligned) load where both are inside the image, bytes otherwise
  uint64_t lo = 0, hi = 0;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int iy = 2 * by + r - pad_t, ix = 2 * bx - pad_l;
    if ((unsigned)iy >= (unsigned)H) continue;
    const int8_t* px = src + ((b * H + iy) * W + ix) * C;
    uint64_t v = 0;
    if (ix >= 0 && ix + 1 < W) {
      __builtin_memcpy(&v, px, 2 * C);
    } else {
#pragma unroll
      for (int dx = 0; dx < 2; ++dx)
        if ((unsigned)(ix + dx) < (unsigned)W) {
#pragma unroll
          for (int c = 0; c < C; ++c) v |= (uint64_t)(uint8_t)px[dx * C + c] << (8 * (dx * C + c));
        }
    }
    constexpr int kBytes = 2 * C;                 // row r lands at bytes [r kBytes, r kBytes + kBytes)
    if (r == 0) {
      lo = v;
    } else if constexpr (kBytes == 8) {
      hi = v;
    } else {
      lo |= v << (8 * kBytes);
      hi = v >> (64 - 8 * kBytes);
    }
  }
  *reinterpret_cast<v4i*>(dst + ((int64_t)b * Hb * Wb + idx) * 16) =
      (v4i){(int)(uint32_t)lo, (int)(uint32_t)(lo >> 32), (int)(uint32_t)hi, (int)(uint32_t)(hi >> 32)};
}

// Both jobs in one launch (jb.B may be 0); C channels in both.
int space_to_depth2_s8(const SpaceToDepthJob& ja, const SpaceToDepthJob& jb, int C, hipStream_t st) {
  const int64_t px = std::max<int64_t>((int64_t)ja.Hb * ja.Wb, (int64_t)jb.Hb * jb.Wb);
  if (px == 0 || ja.B + jb.B == 0) return 0;
  DQ8_REQUIRE(px < (1LL << 31) - 256 && (int64_t)ja.B + jb.B <= 65535 && C >= 1 && C <= 4,
              "space to depth: at most 65535 images of fewer than 2^31 pixels, 1 to 4 channels");
  const dim3 grid((unsigned)ceil_div(px, 256), (unsigned)(ja.B + jb.B));
  auto launch = [&](auto kern) { hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, ja, jb); };
  switch (C) {
    case 1: launch(space_to_depth2_s8_kernel<1>); break;
    case 2: launch(space_to_depth2_s8_kernel<2>); break;
    case 3: launch(space_to_depth2_s8_kernel<3>); break;
    default: launch(space_to_depth2_s8_kernel<4>); break;
  }
  return check_hip(hipGetLastError(), "space-to-depth launch");
}

// int8 [R, C] (row stride ld, any alignment) -> [R, ldd], ldd % 16 == 0 and dst 16-byte
// aligned, columns C .. ldd-1 zero.  One 16-byte store per thread and step.
__global__ void __launch_bounds__(256)
pad_rows_s8_kernel(const int8_t* __restrict__ src, int64_t ld, int8_t* __restrict__ dst,
                   int64_t R, int C, int ldd) {
  const int chunks = ldd / 16;
  const int64_t total = R * chunks;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * 256) {
    const int64_t r = idx / chunks;
    const int c0 = (int)(idx - r * chunks) * 16;
    const int8_t* s = src + r * ld + c0;
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int b = 0; b < 16; ++b)
      if (c0 + b < C) w[b >> 2] |= (uint32_t)(uint8_t)s[b] << (8 * (b & 3));
    *reinterpret_cast<v4i*>(dst + r * ldd + c0) = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  }
}

// out[r] = mul * sum_k X[r, k] + add for an int8 matrix whose rows are 16-byte aligned and a
// multiple of 16 long: the zero-point corrections of a GEMM.  One wave per row.
__global__ void __launch_bounds__(256)
rowsum_s8_kernel(const int8_t* __restrict__ X, int64_t ld, int rows, int K, int mul, int add,
                 int32_t* __restrict__ out) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const v4i* p = reinterpret_cast<const v4i*>(X + (int64_t)row * ld);
  int s = 0;
  for (int c = lane; c < K / 16; c += 64) {
    const v4i v = p[c];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int x = v[w];
      s += (int)(int8_t)x + (int)(int8_t)(x >> 8) + (int)(int8_t)(x >> 16) + (x >> 24);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (lane == 0) out[row] = mul * s + add;
}

#ifdef DQ8_TEST_HOOKS
// one MFMA of each shape, operands straight from global memory
__global__ void __launch_bounds__(64)
mfma_probe_kernel(const int8_t* a, const int8_t* b, int32_t* d32, const int8_t* a16,
                  const int8_t* b16, int32_t* d16) {
  const int lane = threadIdx.x;
  {
    // 32x32x32: lane holds 16 consecutive k of row/column lane%32, k group lane/32
    v4i fa = *(const v4i*)(a + (lane & 31) * 32 + (lane >> 5) * 16);
    v4i fb = *(const v4i*)(b + (lane & 31) * 32 + (lane >> 5) * 16);
    v16i c;
    for (int v = 0; v < 16; ++v) c[v] = 0;
    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, c, 0, 0, 0);
    for (int v = 0; v < 16; ++v) {
      const int i = 8 * (v / 4) + 4 * (lane >> 5) + (v % 4), j = lane & 31;
      d32[i * 32 + j] = c[v];
    }
  }
  {
    // 16x16x64: lane holds 16 consecutive k of row/column lane%16, k group lane/16
    v4i fa = *(const v4i*)(a16 + (lane & 15) * 64 + (lane >> 4) * 16);
    v4i fb = *(const v4i*)(b16 + (lane & 15) * 64 + (lane >> 4) * 16);
    v4i c = {0, 0, 0, 0};
    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa, fb, c, 0, 0, 0);
    for (int v = 0; v < 4; ++v) {
      const int i = 4 * (lane >> 4) + v, j = lane & 15;
      d16[i * 16 + j] = c[v];
    }
  }
}
#endif

// ------------------------------------------------------------- tile variants
// (qgemm_launch.h; every launch_variant<CONV, EPI> is instantiated in a qgemm_launch_*.hip)
}  // namespace
#define DQ8_DECLARE_LAUNCH(CONV, EPI) \
  extern template int launch_variant<CONV, EPI>(int, MainParams&, hipStream_t); \
  extern template int launch_f32a<CONV, EPI>(const MainParams&, hipStream_t); \
  extern template int launch_rowmap<CONV, EPI>(int, MainParams&, hipStream_t);
DQ8_DECLARE_LAUNCH(false, DQ8_EPI_ACC_S32)
DQ8_DECLARE_LAUNCH(false, DQ8_EPI_REQUANT_CPU)
DQ8_DECLARE_LAUNCH(false, DQ8_EPI_REQUANT_GPU)
DQ8_DECLARE_LAUNCH(false, DQ8_EPI_DEQUANT_F32)
DQ8_DECLARE_LAUNCH(true, DQ8_EPI_ACC_S32)
DQ8_DECLARE_LAUNCH(true, DQ8_EPI_REQUANT_CPU)
DQ8_DECLARE_LAUNCH(true, DQ8_EPI_REQUANT_GPU)
DQ8_DECLARE_LAUNCH(true, DQ8_EPI_DEQUANT_F32)
#undef DQ8_DECLARE_LAUNCH

int compute_units() {
  static std::atomic<int> cached{0};
  int v = cached.load(std::memory_order_relaxed);
  if (v > 0) return v;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    (void)hipGetLastError();
    return 256;
  }
  v = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  cached.store(v, std::memory_order_relaxed);
  return v;
}

namespace {

template <bool CONV>
int launch_epi(int variant, MainParams& p, int epilogue, hipStream_t st) {
  switch (epilogue) {
    case DQ8_EPI_ACC_S32: return launch_variant<CONV, DQ8_EPI_ACC_S32>(variant, p, st);
    case DQ8_EPI_REQUANT_CPU: return launch_variant<CONV, DQ8_EPI_REQUANT_CPU>(variant, p, st);
    case DQ8_EPI_REQUANT_GPU: return launch_variant<CONV, DQ8_EPI_REQUANT_GPU>(variant, p, st);
    case DQ8_EPI_DEQUANT_F32: return launch_variant<CONV, DQ8_EPI_DEQUANT_F32>(variant, p, st);
  }
  return fail("unknown epilogue");
}

// (the GEMM over the pixels of a strided 1 x 1 filter; its kernels sit with the convolution's)
int launch_rowmap_epi(int variant, MainParams& p, int epilogue, hipStream_t st) {
  switch (epilogue) {
    case DQ8_EPI_ACC_S32: return launch_rowmap<true, DQ8_EPI_ACC_S32>(variant, p, st);
    case DQ8_EPI_REQUANT_CPU: return launch_rowmap<true, DQ8_EPI_REQUANT_CPU>(variant, p, st);
    case DQ8_EPI_REQUANT_GPU: return launch_rowmap<true, DQ8_EPI_REQUANT_GPU>(variant, p, st);
    case DQ8_EPI_DEQUANT_F32: return launch_rowmap<true, DQ8_EPI_DEQUANT_F32>(variant, p, st);
  }
  return fail("unknown epilogue");
}

// Picks the kernel from the dynamic problem size.  `pipe` says whether the pipelined
// kernels can take the operands.  Measured on BERT-shaped and square problems (M 256 ..
// 16384, N 768 .. 4096, K 768 .. 4096):
//  * the 256x256 tile runs on eight waves (two per SIMD, wave tile 128x64): against four
//    waves of 128x128 the epilogue's chain of VALU instructions per wave halves (5.7 -> 3.1
//    us) and a wave's LDS waits are covered by its neighbour, 3 % at 4096^3 and 10-25 % at
//    K = 768; it pays once its tiles fill about 55 % of the CUs and, past one round of 256
//    tiles, when the last round is not mostly empty (288 tiles = 2 rounds lose to 128x128);
//  * the 128x128 tile from about 120 tiles on -- on eight waves (wave tile 64x32) while
//    K < 4096: 3-20 % faster at K = 768 .. 3072, 2 % slower at K = 4096 --, below that the 64x64 tile spreads the weight
//    stream over more CUs; narrow outputs (N <= 64) take the 256x64 tile.  With 64x64 tiles a
//    CU's operand loads, not its MFMAs, set the pace (16 KiB per 128 of k against 128 MFMA
//    cycles per SIMD); when few CUs are busy and K is deep, splitting K over two wave groups
//    of the workgroup still shortens the chain of dependent k tiles (about 10 % at K = 3072).
//  * 4-byte outputs (int32 sums, f32): the epilogue writes four times as much and, with one
//    256x256 tile per CU, all of it at the very end; while the main loop is short (K < 2048)
//    128x128 tiles, several per CU, write under each other's main loops instead
//    (3072 x 3072 x 768 to f32: 21.8 us against 26.1).
//  * int8 output, big tiles: 256x256 against 256x192 (wave tile 64x96), one-shot against
//    persistent.  Measured per workgroup with all compute units busy and K = 768: 1.8 us until
//    the first k tile has landed, 1.6 us (256x256) or 1.27 us (256x192) per k tile, 2.8 / 2.1 us
//    of requantisation (4 VALU instructions per result at 4 cycles each per SIMD: bound by the
//    vector ALU), 0.75 us before the next workgroup starts on the compute unit.  The matrix
//    pipe is power-limited: a k tile takes 1.0 us with a few compute units busy and 1.65 us
//    with all 256, which is why a shape that fills 192 compute units with 256x256 tiles gains
//    only 6-10 % from 256 tiles of 256x192 and not the 25 % its idle quarter suggests.  The
//    persistent form saves the first-tile latency and the hand-over (1.5 us per tile) from
//    the second tile of a workgroup on and costs about 1 us per launch.
// 64 x 64 tiles with the k range split inside the workgroup: over two wave groups, and over
// four from 8192 of k on while there is at most a tile per compute unit (M = 128,
// 11008 -> 4096: 20.8 against 23.4 us; M = 32, 8192^2: 17.1 against 18.8; M = 256, 16384 -> 1024:
// 25.4 against 30.7; at 3072 of k the wider reduction costs more than the shorter loop saves)
int pick_k_split64(int64_t M, int64_t N, int64_t K) {
  const int64_t t64 = ceil_div(M, 64) * ceil_div(N, 64);
  return (K >= 8192 && t64 <= compute_units()) ? kPipe64k4 : kPipe64k2;
}

int pick_variant(int64_t M, int64_t N, int64_t K, bool pipe, int out_bytes = 1) {
  auto tiles = [&](int v) { return ceil_div(M, kVariants[v].bm) * ceil_div(N, kVariants[v].bn); };
  if (pipe) {
    const int64_t cus = compute_units();
    // (256 x 64 tiles for a narrow N once they occupy three quarters of the compute units)
    if (N <= 64 && 4 * tiles(kPipe256x64) >= 3 * cus) return kPipe256x64;
    // A wide tile is a candidate while at least 0.7 of the columns of its tiles are columns of
    // the problem (M = 100352, 256 -> 128: 256 x 192 tiles 14.6 us, 128 x 128 12.9; M = 25088,
    // 512 -> 256: 10.9 against 8.9).
    auto columns_used = [&](int v) { return 10 * N >= 7 * ceil_div(N, kVariants[v].bn) * kVariants[v].bn; };
    const int64_t t256 = tiles(kPipe256w8);
    const int64_t rounds = ceil_div(t256, cus);
    const bool big256 = t256 >= 140 && (rounds == 1 || 10 * t256 >= 7 * cus * rounds) &&
                        (out_bytes == 1 || K >= 2048) && columns_used(kPipe256w8);
    if (out_bytes == 1) {
      // estimated time in us of a launch of `t` tiles whose k tile costs `per_k` us with all
      // compute units busy and whose fixed parts cost `fixed` us
      const double kt = (double)ceil_div(K, 128);
      auto estimate = [&](int64_t t, double per_k, double fixed, bool* persistent) {
        const int64_t r = ceil_div(t, cus);
        const double busy = (double)(t < cus ? t : cus) / (double)cus;
        const double throttle = (1.0 + 0.65 * busy * std::sqrt(busy)) / 1.65;
        *persistent = r >= 2;
        return (double)r * (kt * per_k * throttle + fixed) - (*persistent ? (double)(r - 1) * 1.5 - 1.0 : 0.0);
      };
      const int64_t t192 = tiles(kPipe256x192);
      bool p256 = false, p192 = false;
      const double e256 = big256 ? estimate(t256, 1.6, 5.4, &p256) : 1e30;
      // (from 180 tiles: M = 1152, 2048 -> 7424, 195 tiles: 24.3 against 27.2 us on 145 of 256 x 256)
      const double e192 = t192 >= 180 && columns_used(kPipe256x192) ? estimate(t192, 1.27, 4.7, &p192) : 1e30;
      if (e192 < e256) return p192 ? kPersist256x192 : kPipe256x192;
      if (big256) return p256 ? kPersist256 : kPipe256w8;
    } else if (big256) {
      return kPipe256w8;
    }
    // 128x128: eight waves while every tile has a compute unit to itself (more waves to cover
    // the load latency: 6.3 against 7.1 us at M = 2048, 768 -> 768); with two tiles on a
    // compute unit, or a deep K, four waves (10.0 against 11.2 us at M = 2048, 768 -> 3072)
    const int64_t t128 = tiles(kPipe128);
    // 128 x 128 tiles, two to a compute unit, that end in a round of a few tiles (at most a
    // quarter of a round) pay a whole k loop for them: the larger tiles, whichever the estimate
    // prefers, although they leave compute units idle (M = 768, 4096 -> 11008: 516 tiles of
    // 128 x 128 55.1 us, 174 of 256 x 192 38.4)
    if (out_bytes == 1 && t128 > 2 * cus && t128 % (2 * cus) != 0 && t128 % (2 * cus) <= cus / 2) {
      const double kt = (double)ceil_div(K, 128);
      auto one_round = [&](int64_t t, double per_k, double fixed) {
        const double busy = (double)(t < cus ? t : cus) / (double)cus;
        return (double)ceil_div(t, cus) * (kt * per_k * (1.0 + 0.65 * busy * std::sqrt(busy)) / 1.65 + fixed);
      };
      const int64_t t192 = tiles(kPipe256x192);
      if (t256 <= cus && t192 <= cus && columns_used(kPipe256x192) && columns_used(kPipe256w8))
        return one_round(t192, 1.27, 4.7) < one_round(t256, 1.6, 5.4) ? kPipe256x192 : kPipe256w8;
    }
    // (int32 / f32 results, four times the bytes to store: eight waves throughout, and the
    // persistent form from two tiles per compute unit on -- M = 16384, 768 -> 768 with an f32
    // result: 17.8 against 18.5 us, four waves 23.8)
    if (t128 >= 120) {
      // (deep K: four waves; while the 128 x 128 tiles leave compute units idle and the 64 x 64
      // ones come to at most two per unit, those with the k range split over two wave groups --
      // M = 256, 8192^2 weights: 28.5 against 33.1 us; M = 512, 4096^2: 16.4 against 18.0)
      if (K >= 4096)
        return (t128 < cus && tiles(kPipe64) <= 2 * cus) ? pick_k_split64(M, N, K) : kPipe128;
      if (out_bytes == 1) return t128 <= cus ? kPipe128w8 : kPipe128;
      return t128 > 2 * cus ? kPersist128 : kPipe128w8;
    }
    // (64 x 64 tiles: the k range split over two wave groups while they come to at most one per
    // compute unit, from 4096 of k on at most two -- M = 384, 11008 -> 4096: 37.0 against 40.1 us)
    return (K >= 2048 && tiles(kPipe64) <= (K >= 4096 ? 2 * cus : cus)) ? pick_k_split64(M, N, K)
                                                                        : kPipe64;
  }
  // (operands the pipelined kernels cannot address: the 128 x 128 and 64 x 64 tiles of the basic
  // kernel; its 256 x 256 form on four waves indexes 256 accumulators per lane and is kept
  // only as a cross-check variant)
  const int64_t cus = compute_units();
  if (tiles(2) >= cus - cus / 8) return 2;
  return 3;
}

// The small-M kernel up to kSkinnyMaxM rows -- except against weights wide enough to give the
// 64 x 64 tile with its k range split over two wave groups a workgroup for every second compute
// unit or more: its time hardly depends on M, the small-M kernel's grows with it.  From 17 rows
// at 128 tiles (M = 32, 8192 x 8192 weights: 18.5 against 24.6 us; 4096 x 4096: 9.1 against
// 8.5), from 9 rows at 144 (M = 16, 4096 -> 11008: 12.0 against 14.2 us; at 128 tiles, 8192^2,
// 18.7 against 17.9), from 3 rows at 224 (M = 4, 4096 -> 16384: 13.2 against 15.1 us; M = 16,
// 8192 -> 16384: 22.0 against 32.0) -- and the tiled kernels above.
int pick_any(int64_t M, int64_t N, int64_t K, bool pipe, int out_bytes) {
  if (M <= kSkinnyMaxM) {
    const int64_t t64 = ceil_div(N, 64);
    if (pipe && K >= 2048 &&
        ((M > 16 && t64 >= 128) || (M >= 9 && t64 >= 144) || (M >= 3 && t64 >= 224)))
      return pick_k_split64(M, N, K);
    return kSkinnyVariant;
  }
  if (skinny_takes_rows(M, N, K)) return kSkinnyVariant;
  return pick_variant(M, N, K, pipe, out_bytes);
}

// Whether a 3x3 stride-1 convolution goes to the kernel that keeps the input patch in LDS
// (and with which tile), or to the implicit GEMM.  Measured on ResNet / VGG shaped layers
// with batch 1 .. 128: with at most 64 input and output channels the implicit GEMM is bound
// by its operand loads (each input pixel is fetched nine times) and the direct kernel wins
// by 12-30 % once its 256-pixel tiles fill the chip; with more channels the implicit GEMM's
// larger tiles are as fast or faster.  Returns the configuration or -1.
int pick_direct_conv(int64_t images, int64_t pixels_per_image, int64_t Ci, int64_t Co) {
  if (Ci > 64 || Co > 64) return -1;
  int bm, bn;
  // 512-pixel tiles on eight waves when they give every compute unit at most one workgroup
  // and leave few idle: one round, no second workgroup competing for the matrix pipe
  // (32 x 56 x 56 x 64 -> 64: 224 workgroups, 9.2 against 9.9 us)
  direct_conv_tile(2, &bm, &bn);
  const int64_t cus = compute_units();
  const int64_t wg512 = images * ceil_div(pixels_per_image, bm) * ceil_div(Co, bn);
  if (wg512 <= cus && 4 * wg512 >= 3 * cus) return 2;
  // else the largest of the 256- and 128-pixel tiles that still occupies three quarters of
  // the compute units (batch 8 of the same layer: 200 workgroups of 128 pixels 6.5 us, 104 of
  // 256 pixels 7.8, the implicit GEMM's 256 x 64 tiles 9.4)
  for (int config : {0, 1}) {
    direct_conv_tile(config, &bm, &bn);
    if (4 * images * ceil_div(pixels_per_image, bm) * ceil_div(Co, bn) >= 3 * cus) return config;
  }
  return -1;
}

int elem_size(int epilogue) {
  return (epilogue == DQ8_EPI_ACC_S32 || epilogue == DQ8_EPI_DEQUANT_F32) ? 4 : 1;
}

int check_epilogue(const char* who, int epilogue, const void* bias, int bias_kind,
                   const float* sx, const float* sw, const float* so, int64_t n_sx,
                   int64_t n_sw, int64_t n_so, int64_t N) {
  const std::string w(who);
  DQ8_REQUIRE(epilogue >= DQ8_EPI_ACC_S32 && epilogue <= DQ8_EPI_DEQUANT_F32,
              w + ": unknown epilogue");
  DQ8_REQUIRE(bias_kind >= DQ8_BIAS_NONE && bias_kind <= DQ8_BIAS_S8,
              w + ": unknown bias kind");
  DQ8_REQUIRE((bias_kind == DQ8_BIAS_NONE) == (bias == nullptr) ||
                  (bias_kind == DQ8_BIAS_NONE),
              w + ": bias pointer missing");
  if (epilogue == DQ8_EPI_ACC_S32) {
    DQ8_REQUIRE(bias_kind == DQ8_BIAS_NONE, w + ": ACC_S32 takes no bias");
    return 0;
  }
  DQ8_REQUIRE(sx && sw, w + ": scale pointer missing");
  DQ8_REQUIRE((n_sx == 1 || n_sx == N) && (n_sw == 1 || n_sw == N),
              w + ": scale vectors must have 1 or N entries");
  if (epilogue == DQ8_EPI_DEQUANT_F32) {
    DQ8_REQUIRE(bias_kind == DQ8_BIAS_NONE || bias_kind == DQ8_BIAS_F32,
                w + ": DEQUANT_F32 takes an f32 bias or none");
    return 0;
  }
  DQ8_REQUIRE(so && (n_so == 1 || n_so == N), w + ": output scale missing or mis-sized");
  if (epilogue == DQ8_EPI_REQUANT_CPU)
    DQ8_REQUIRE(bias_kind != DQ8_BIAS_S8, w + ": REQUANT_CPU takes s32/f32 bias or none");
  if (epilogue == DQ8_EPI_REQUANT_GPU)
    DQ8_REQUIRE(bias_kind != DQ8_BIAS_S32, w + ": REQUANT_GPU takes f32/s8 bias or none");
  return 0;
}

// Validates the fused operators against the epilogue and puts them into the kernel
// parameters.  `int8_out`: the epilogue proper writes int8; `n_so`: entries of the output scale.
int apply_postops(const char* who, const dq8_postops_t* post, bool int8_out, bool f32_requant,
                  int64_t n_so, int64_t N, EpiParams* e) {
  if (!post || (post->residual_kind == DQ8_RESIDUAL_NONE && !post->table)) return 0;
  const std::string w(who);
  DQ8_REQUIRE(int8_out || f32_requant,
              w + ": fused operators need a requantising epilogue");
  if (post->table) {
    DQ8_REQUIRE(int8_out && post->residual_kind == DQ8_RESIDUAL_NONE,
                w + ": a fused table takes an int8 result and no residual");
    e->table = static_cast<const uint8_t*>(post->table);
    return 0;
  }
  DQ8_REQUIRE(post->residual_kind == DQ8_RESIDUAL_F32 || post->residual_kind == DQ8_RESIDUAL_S8,
              w + ": unknown residual kind");
  DQ8_REQUIRE(post->residual != nullptr && post->ldr >= N, w + ": residual missing or too narrow");
  DQ8_REQUIRE(n_so == 1, w + ": a fused residual takes a per-tensor output scale");
  DQ8_REQUIRE(post->residual_kind != DQ8_RESIDUAL_S8 || post->residual_scale != nullptr,
              w + ": an int8 residual needs its scale");
  DQ8_REQUIRE(int8_out == (post->out_scale != nullptr),
              w + ": int8 results with a residual need out_scale, f32 results take none");
  e->resid = post->residual;
  e->resid_kind = post->residual_kind;
  e->ldr = post->ldr;
  e->resid_scale = post->residual_scale;
  e->resid_zp = post->residual_zp;
  e->relu = post->relu != 0;
  e->out_scale = post->out_scale;
  e->out_zp = post->out_zp;
  const int esz = post->residual_kind == DQ8_RESIDUAL_F32 ? 4 : 1;
  e->resid_vec = aligned(post->residual, 16) && (post->ldr * esz) % 16 == 0;
  return 0;
}

template <typename P>
int launch_generic_epi(void (*k0)(const P), void (*k1)(const P), void (*k2)(const P),
                       void (*k3)(const P), int epilogue, const P& p, int64_t total,
                       hipStream_t st) {
  int64_t blocks = std::min<int64_t>(ceil_div(total, 256), 256 * 32);
  void (*k)(const P) = epilogue == DQ8_EPI_ACC_S32       ? k0
                       : epilogue == DQ8_EPI_REQUANT_CPU ? k1
                       : epilogue == DQ8_EPI_REQUANT_GPU ? k2
                                                         : k3;
  hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), 0, st, p);
  return check_hip(hipGetLastError(), "generic kernel launch");
}

}  // namespace
}  // namespace dq8

using namespace dq8;

#ifdef DQ8_TEST_HOOKS   // (tests/dq8_test_hooks.h; compiled into libdisc_q8_testhooks.so only)
extern "C" int dq8_qgemm_num_variants(void) { return kNumVariants; }

extern "C" const char* dq8_qgemm_variant_name(int variant) {
  if (variant < 0 || variant >= kNumVariants) return "";
  return kVariants[variant].name;
}
#endif

extern "C" size_t dq8_qgemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int tp_a,
                                            int tp_b) {
  // an operand that is not k-contiguous, or whose K is not a multiple of 16, is rewritten
  // as [rows, K rounded up to 16] (zero filled) for the MFMA kernels
  size_t bytes = 0;
  auto pad = [](int64_t v) { return (size_t)((v + 255) / 256 * 256); };
  const int64_t kp = (K + 15) / 16 * 16;
  if (tp_a || K % 16 != 0) bytes += pad(M * kp);
  if (!tp_b || K % 16 != 0) bytes += pad(N * kp);
  return bytes;
}

extern "C" size_t dq8_qgemm_workspace_bytes_zp(int64_t M, int64_t N, int64_t K, int tp_a,
                                               int tp_b, int32_t zx, int32_t zw) {
  size_t bytes = dq8_qgemm_workspace_bytes(M, N, K, tp_a, tp_b);
  if (zx != 0 || zw != 0) {   // the per-column and per-row corrections
    auto pad = [](int64_t v) { return (size_t)((v + 255) / 256 * 256); };
    bytes += pad(N * 4) + pad(M * 4);
  }
  return bytes;
}

extern "C" int dq8_transpose_s8(const int8_t* src, int64_t ld, int8_t* dst, int64_t rows,
                                int64_t cols, void* stream) {
  clear_error();
  DQ8_REQUIRE(rows >= 0 && cols >= 0 && ld >= cols, "dq8_transpose_s8: bad shape");
  DQ8_REQUIRE(rows < (1LL << 31) && cols < (1LL << 31), "dq8_transpose_s8: too large");
  if (rows == 0 || cols == 0) return 0;
  DQ8_REQUIRE(src && dst, "dq8_transpose_s8: null pointer");
  hipLaunchKernelGGL(transpose_s8_kernel,
                     dim3((unsigned)ceil_div(cols, 64), (unsigned)ceil_div(rows, 64)), dim3(256),
                     0, (hipStream_t)stream, src, ld, dst, (int)rows, (int)cols, (int)rows);
  return check_hip(hipGetLastError(), "dq8_transpose_s8 launch");
}

namespace {
int qgemm_impl(int variant, const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw, void* out,
               int64_t ldo, int64_t M, int64_t N, int64_t K, int tp_a, int tp_b, int epilogue,
               const void* bias, int bias_kind, const float* sx, int64_t n_sx, const float* sw,
               int64_t n_sw, const float* so, int64_t n_so, int32_t zx, int32_t zw, int32_t zo,
               void* workspace, size_t workspace_bytes, const dq8_postops_t* post, void* stream) {
  clear_error();
  DQ8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "dq8_qgemm: negative size");
  DQ8_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K < (1LL << 31),
              "dq8_qgemm: dimension exceeds 2^31-1");
  DQ8_REQUIRE(variant >= -1 && variant < kNumVariants, "dq8_qgemm: unknown variant");
  // requant -> dequantize in one epilogue: validated as the requant form it starts with,
  // run by the f32-output kernels
  int requant = 0;
  if (epilogue == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 || epilogue == DQ8_EPI_REQUANT_GPU_DEQUANT_F32) {
    requant = epilogue == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 ? 1 : 2;
    DQ8_REQUIRE(n_so == 1, "dq8_qgemm: the requant -> dequantize epilogues take a per-tensor "
                           "output scale");
    epilogue = requant == 1 ? DQ8_EPI_REQUANT_CPU : DQ8_EPI_REQUANT_GPU;
  }
  int fixedpoint = 0;
  if (epilogue == DQ8_EPI_REQUANT_FIXEDPOINT) {
    fixedpoint = 1;
    DQ8_REQUIRE(n_sx == 1 && n_so == 1, "dq8_qgemm: the fixed-point stage takes per-tensor input "
                                        "and output scales");
    DQ8_REQUIRE(bias_kind == DQ8_BIAS_NONE || bias_kind == DQ8_BIAS_S32,
                "dq8_qgemm: the fixed-point stage takes an s32 bias or none");
    epilogue = DQ8_EPI_REQUANT_CPU;
  }
  if (int s = check_epilogue("dq8_qgemm", epilogue, bias, bias_kind, sx, sw, so, n_sx,
                             n_sw, n_so, N))
    return s;
  DQ8_REQUIRE(zo == 0 || epilogue == DQ8_EPI_REQUANT_CPU,
              "dq8_qgemm: an output zero point needs the REQUANT_CPU epilogue");
  if (requant) epilogue = DQ8_EPI_DEQUANT_F32;
  if (M == 0 || N == 0) return 0;
  DQ8_REQUIRE(out != nullptr, "dq8_qgemm: null output");
  DQ8_REQUIRE(K == 0 || (A && W), "dq8_qgemm: null operand");
  DQ8_REQUIRE(lda >= (tp_a ? M : K) && ldw >= (tp_b ? K : N) && ldo >= N,
              "dq8_qgemm: leading dimension smaller than the row length");
  hipStream_t st = (hipStream_t)stream;

  EpiParams e = {};
  e.out = out;
  e.ldo = ldo;
  e.M = (int)M;
  e.N = (int)N;
  e.bias = bias;
  e.bias_kind = bias_kind;
  e.sx = sx;
  e.sw = sw;
  e.so = so;
  e.sx_stride = n_sx > 1;
  e.sw_stride = n_sw > 1;
  e.so_stride = n_so > 1;
  e.zo = zo;
  e.requant = requant;
  e.fixedpoint = fixedpoint;
  const int es = elem_size(epilogue);
  e.vec_store = aligned(out, 4 * es) && (ldo % 4 == 0);
  e.vec_store16 = aligned(out, 16) && (ldo % 16 == 0);
  if (int s = apply_postops("dq8_qgemm", post, es == 1 && epilogue != DQ8_EPI_ACC_S32, requant != 0,
                            n_so, N, &e))
    return s;

  // Zero points: sum (a - zx)(w - zw) = sum a w - zx SW[n] - zw SA[m] + K zx zw with the row
  // sums SW, SA.  Given scratch for the two correction vectors the heuristic keeps the
  // problem on the pipelined MFMA kernels, whose accumulators start at the corrections;
  // otherwise (or for operands those kernels cannot take) the generic kernel subtracts the
  // zero points itself.
  const bool has_zp = zx != 0 || zw != 0;
  const bool auto_pick = variant == -1;
  // The MFMA kernels want A [M, K'] and W [N, K'], k-contiguous, rows 16-byte aligned, K' a
  // multiple of 16: operands in another layout, or with a ragged K, are rewritten into the
  // workspace (zero-filled up to K'; zeros add nothing to the sums).
  const int64_t Kp = (K + 15) / 16 * 16;
  const bool repack_a = K > 0 && (tp_a || K % 16 != 0);
  const bool repack_w = K > 0 && (!tp_b || K % 16 != 0);
  const bool have_ws = workspace != nullptr && aligned(workspace, 256) &&
                       workspace_bytes >= dq8_qgemm_workspace_bytes(M, N, K, tp_a, tp_b);
  const bool mfma_operands = (repack_a ? have_ws : (aligned(A, 16) && lda % 16 == 0)) &&
                             (repack_w ? have_ws : (aligned(W, 16) && ldw % 16 == 0));
  const bool zp_mfma =
      has_zp && auto_pick && K > 0 && mfma_operands && workspace != nullptr &&
      aligned(workspace, 256) &&
      workspace_bytes >= dq8_qgemm_workspace_bytes_zp(M, N, K, tp_a, tp_b, zx, zw);
  if (auto_pick && has_zp && !zp_mfma) variant = 0;
  // fused operators are implemented on the vector store paths of the MFMA kernels (and in
  // the generic kernel): output rows that are not 16-byte aligned take the generic kernel
  const bool fused = e.table != nullptr || e.resid_kind != 0;
  if (fused && !(es == 1 ? e.vec_store16 : e.vec_store)) variant = 0;
  // (a ragged K without the scratch to pad it, or unaligned operands: the generic kernel
  // takes any strides; a transposed operand without scratch stays an error below)
  if (variant != 0 && !mfma_operands && !((tp_a || !tp_b) && !have_ws)) variant = 0;
  if (variant == 0) {
    GenericParams g;
    g.A = A;
    g.W = W;
    g.a_sm = tp_a ? 1 : lda;
    g.a_sk = tp_a ? lda : 1;
    g.w_sn = tp_b ? ldw : 1;
    g.w_sk = tp_b ? 1 : ldw;
    g.K = (int)K;
    g.zx = zx;
    g.zw = zw;
    g.epi = e;
    return launch_generic_epi<GenericParams>(
        qgemm_generic_kernel<DQ8_EPI_ACC_S32>, qgemm_generic_kernel<DQ8_EPI_REQUANT_CPU>,
        qgemm_generic_kernel<DQ8_EPI_REQUANT_GPU>, qgemm_generic_kernel<DQ8_EPI_DEQUANT_F32>,
        epilogue, g, M * N, st);
  }
  DQ8_REQUIRE(!has_zp || zp_mfma,
              "dq8_qgemm: input/weight zero points need the heuristic (variant -1) or the "
              "generic variant");
  DQ8_REQUIRE(mfma_operands, "dq8_qgemm: workspace too small for the requested transposes");

  const int8_t* a_use = A;
  const int8_t* w_use = W;
  int64_t lda_use = lda, ldw_use = ldw;
  size_t ws_off = 0;
  auto pad = [](int64_t v) { return (size_t)((v + 255) / 256 * 256); };
  auto repack = [&](const int8_t* src, int64_t ld, bool transposed, int64_t rows) {
    int8_t* dst = (int8_t*)workspace + ws_off;
    if (transposed)   // src is [K, rows]
      hipLaunchKernelGGL(transpose_s8_kernel,
                         dim3((unsigned)ceil_div(rows, 64), (unsigned)ceil_div(Kp, 64)), dim3(256),
                         0, st, src, ld, dst, (int)K, (int)rows, (int)Kp);
    else
      hipLaunchKernelGGL(pad_rows_s8_kernel,
                         dim3((unsigned)std::min<int64_t>(ceil_div(rows * (Kp / 16), 256), 1 << 20)),
                         dim3(256), 0, st, src, ld, dst, rows, (int)K, (int)Kp);
    ws_off += pad(rows * Kp);
    return dst;
  };
  if (repack_a) {
    a_use = repack(A, lda, tp_a != 0, M);
    lda_use = Kp;
  }
  if (repack_w) {
    w_use = repack(W, ldw, tp_b == 0, N);
    ldw_use = Kp;
  }
  if (repack_a || repack_w) DQ8_HIP(hipGetLastError());
  const int64_t K_true = K;
  K = Kp;   // what the kernels below see; the padding is zero

  MainParams p = {};
  p.A = a_use;
  p.W = w_use;
  p.lda = lda_use;
  p.ldw = ldw_use;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.epi = e;
  if (auto_pick)
    variant = pick_any(M, N, K, pipe_ok(256, 256, p, false), es);
  if (fused || e.fixedpoint) {   // the persistent forms carry neither
    DQ8_REQUIRE(auto_pick || (variant != kPersist256 && variant != kPersist256x192 && variant != kPersist128),
                "dq8_qgemm: the persistent variants take neither fused operators nor the fixed-point stage");
    if (variant == kPersist256) variant = kPipe256w8;
    if (variant == kPersist256x192) variant = kPipe256x192;
    if (variant == kPersist128) variant = kPipe128w8;
  }
  if (!zp_mfma) return launch_epi<false>(variant, p, epilogue, st);

  // ---- zero points: row sums -> corrections -> a pipelined kernel that starts from them
  if (!is_pipe_variant(variant)) variant = kPipe64;   // (small M, or tiles the others cannot address)
  if (!pipe_ok(kVariants[variant].bm, kVariants[variant].bn, p, false)) {
    GenericParams g;
    g.A = a_use;
    g.W = w_use;
    g.a_sm = lda_use;
    g.a_sk = 1;
    g.w_sn = ldw_use;
    g.w_sk = 1;
    g.K = (int)K_true;   // (the padding is not part of the sums)
    g.zx = zx;
    g.zw = zw;
    g.epi = e;
    return launch_generic_epi<GenericParams>(
        qgemm_generic_kernel<DQ8_EPI_ACC_S32>, qgemm_generic_kernel<DQ8_EPI_REQUANT_CPU>,
        qgemm_generic_kernel<DQ8_EPI_REQUANT_GPU>, qgemm_generic_kernel<DQ8_EPI_DEQUANT_F32>,
        epilogue, g, M * N, st);
  }
  int32_t* corr_n = reinterpret_cast<int32_t*>((int8_t*)workspace + ws_off);
  int32_t* corr_m = reinterpret_cast<int32_t*>((int8_t*)corr_n + pad(N * 4));
  // (wrapping int32 arithmetic on purpose, as in the kernels)
  const int kzz = (int)((uint32_t)K_true * (uint32_t)zx * (uint32_t)zw);
  hipLaunchKernelGGL(rowsum_s8_kernel, dim3((unsigned)ceil_div(N, 4)), dim3(256), 0, st, w_use,
                     ldw_use, (int)N, (int)K, -zx, kzz, corr_n);
  if (zw != 0)
    hipLaunchKernelGGL(rowsum_s8_kernel, dim3((unsigned)ceil_div(M, 4)), dim3(256), 0, st, a_use,
                       lda_use, (int)M, (int)K, -zw, 0, corr_m);
  DQ8_HIP(hipGetLastError());
  p.corr_n = corr_n;
  p.corr_m = zw != 0 ? corr_m : nullptr;
  return launch_epi<false>(variant, p, epilogue, st);
}
}  // namespace

extern "C" const char* dq8_qgemm_kernel_name(int64_t M, int64_t N, int64_t K, int out_bytes) {
  if (M <= 0 || N <= 0 || K <= 0 || M >= (1LL << 31) || N >= (1LL << 31) || K >= (1LL << 31))
    return "";
  if (K % 16 != 0) return kVariants[0].name;
  MainParams p = {};
  p.lda = p.ldw = K;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  return kVariants[pick_any(M, N, K, pipe_ok(256, 256, p, false), out_bytes == 1 ? 1 : 4)].name;
}

#ifdef DQ8_TEST_HOOKS
extern "C" int dq8_qgemm_variant(int variant, const int8_t* A, int64_t lda,
                                 const int8_t* W, int64_t ldw, void* out, int64_t ldo,
                                 int64_t M, int64_t N, int64_t K, int tp_a, int tp_b,
                                 int epilogue, const void* bias, int bias_kind,
                                 const float* sx, int64_t n_sx, const float* sw,
                                 int64_t n_sw, const float* so, int64_t n_so,
                                 int32_t zx, int32_t zw, int32_t zo, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  return qgemm_impl(variant, A, lda, W, ldw, out, ldo, M, N, K, tp_a, tp_b, epilogue, bias,
                    bias_kind, sx, n_sx, sw, n_sw, so, n_so, zx, zw, zo, workspace,
                    workspace_bytes, nullptr, stream);
}
#endif

extern "C" int dq8_qgemm_fused(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw,
                               void* out, int64_t ldo, int64_t M, int64_t N, int64_t K, int tp_a,
                               int tp_b, int epilogue, const void* bias, int bias_kind,
                               const float* sx, int64_t n_sx, const float* sw, int64_t n_sw,
                               const float* so, int64_t n_so, int32_t zx, int32_t zw, int32_t zo,
                               void* workspace, size_t workspace_bytes,
                               const dq8_postops_t* post, void* stream) {
  return qgemm_impl(-1, A, lda, W, ldw, out, ldo, M, N, K, tp_a, tp_b, epilogue, bias, bias_kind,
                    sx, n_sx, sw, n_sw, so, n_so, zx, zw, zo, workspace, workspace_bytes, post,
                    stream);
}

extern "C" int dq8_qgemm(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw,
                         void* out, int64_t ldo, int64_t M, int64_t N, int64_t K,
                         int tp_a, int tp_b, int epilogue, const void* bias,
                         int bias_kind, const float* sx, int64_t n_sx, const float* sw,
                         int64_t n_sw, const float* so, int64_t n_so, int32_t zx,
                         int32_t zw, int32_t zo, void* workspace, size_t workspace_bytes,
                         void* stream) {
  return qgemm_impl(-1, A, lda, W, ldw, out, ldo, M, N, K, tp_a, tp_b, epilogue, bias, bias_kind,
                    sx, n_sx, sw, n_sw, so, n_so, zx, zw, zo, workspace, workspace_bytes, nullptr,
                    stream);
}

// ---- quantize -> qgemm as one operator ---------------------------------------------------
extern "C" int64_t dq8_qlinear_f32_fused_max_rows(int64_t N, int64_t K) {
  // A workgroup takes 16 rows x 16 channels, and every workgroup along N quantizes its 16 rows
  // again.  That is cheaper than a quantize launch of its own (about 2.2 us) while the
  // workgroups come to at most three per compute unit (one per compute unit from 3072 of k
  // on).  Measured against dq8_quantize + dq8_qgemm with the dequantize in its epilogue
  // (launches replayed from a graph, us): 768 -> 768: 16 rows 4.1 against 5.4, 64 rows 4.2 / 7.9,
  // 256 rows 6.0 / 8.3, 512 rows 9.4 / 8.3; 768 -> 2304: 64 rows 6.0 / 8.0, 128 rows 8.3 / 8.2;
  // 768 -> 3072: 64 rows 6.1 / 8.1, 128 rows 9.4 / 8.1; 3072 -> 768: 64 rows 6.5 / 11.4, 256 rows
  // 11.2 / 12.3, 512 rows 21.3 / 13.0; 4096 -> 4096: 16 rows 9.1 / 9.2, 32 rows 12.3 / 11.4.
  if (N <= 0 || N >= (1LL << 31) || K < 16 || K % 16 != 0) return 0;
  const int64_t cus = compute_units();
  const int64_t blocks = (K <= 3072 ? 3 * cus : cus) / ceil_div(N, 16);
  return std::min<int64_t>(16 * blocks, 4096);
}

extern "C" int dq8_qlinear_f32(const float* X, int64_t ldx, const int8_t* W, int64_t ldw, void* out,
                               int64_t ldo, int64_t M, int64_t N, int64_t K, int epilogue,
                               const void* bias, int bias_kind, const float* sx, const float* sw,
                               int64_t n_sw, const float* so, int64_t n_so, int32_t zo,
                               int round_mode, void* stream) {
  clear_error();
  DQ8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "dq8_qlinear_f32: negative size");
  DQ8_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K < (1LL << 31), "dq8_qlinear_f32: 2^31 limit");
  DQ8_REQUIRE(round_mode == DQ8_ROUND_HALF_TO_EVEN || round_mode == DQ8_ROUND_HALF_AWAY_FROM_ZERO,
              "dq8_qlinear_f32: unknown round_mode");
  DQ8_REQUIRE(epilogue != DQ8_EPI_REQUANT_FIXEDPOINT,
              "dq8_qlinear_f32: the fixed-point stage is not offered here");
  if (M == 0 || N == 0) return 0;
  DQ8_REQUIRE(X && sx, "dq8_qlinear_f32: null activations or scale");
  DQ8_REQUIRE(ldx >= K, "dq8_qlinear_f32: leading dimension smaller than the row length");
  hipStream_t st = (hipStream_t)stream;
  DQ8_REQUIRE(M <= dq8_qlinear_f32_fused_max_rows(N, K),
              "dq8_qlinear_f32: more rows than dq8_qlinear_f32_fused_max_rows() (or K % 16 != 0): "
              "run dq8_quantize and dq8_qgemm");
  DQ8_REQUIRE(aligned(X, 16) && ldx % 4 == 0 && aligned(W, 16) && ldw % 16 == 0,
              "dq8_qlinear_f32: rows of X and W must be 16-byte aligned");
  // the same validation and epilogue set-up as dq8_qgemm
  int requant = 0;
  if (epilogue == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 || epilogue == DQ8_EPI_REQUANT_GPU_DEQUANT_F32) {
    requant = epilogue == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 ? 1 : 2;
    epilogue = requant == 1 ? DQ8_EPI_REQUANT_CPU : DQ8_EPI_REQUANT_GPU;
  }
  if (int s = check_epilogue("dq8_qlinear_f32", epilogue, bias, bias_kind, sx, sw, so, 1, n_sw,
                             n_so, N))
    return s;
  DQ8_REQUIRE(zo == 0 || epilogue == DQ8_EPI_REQUANT_CPU,
              "dq8_qlinear_f32: an output zero point needs the REQUANT_CPU epilogue");
  if (requant) epilogue = DQ8_EPI_DEQUANT_F32;
  DQ8_REQUIRE(out != nullptr && W != nullptr, "dq8_qlinear_f32: null pointer");
  DQ8_REQUIRE(ldw >= K && ldo >= N, "dq8_qlinear_f32: leading dimension smaller than the row length");
  MainParams p = {};
  p.A = reinterpret_cast<const int8_t*>(X);
  p.W = W;
  p.lda = ldx;
  p.ldw = ldw;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.a_scale = sx;
  p.a_round_even = round_mode == DQ8_ROUND_HALF_TO_EVEN;
  EpiParams& e = p.epi;
  e.out = out;
  e.ldo = ldo;
  e.M = (int)M;
  e.N = (int)N;
  e.bias = bias;
  e.bias_kind = bias_kind;
  e.sx = sx;
  e.sw = sw;
  e.so = so;
  e.sx_stride = 0;
  e.sw_stride = n_sw > 1;
  e.so_stride = n_so > 1;
  e.zo = zo;
  e.requant = requant;
  const int es = elem_size(epilogue);
  e.vec_store = aligned(out, 4 * es) && (ldo % 4 == 0);
  e.vec_store16 = aligned(out, 16) && (ldo % 16 == 0);
  switch (epilogue) {
    case DQ8_EPI_ACC_S32: return launch_f32a<false, DQ8_EPI_ACC_S32>(p, st);
    case DQ8_EPI_REQUANT_CPU: return launch_f32a<false, DQ8_EPI_REQUANT_CPU>(p, st);
    case DQ8_EPI_REQUANT_GPU: return launch_f32a<false, DQ8_EPI_REQUANT_GPU>(p, st);
    case DQ8_EPI_DEQUANT_F32: return launch_f32a<false, DQ8_EPI_DEQUANT_F32>(p, st);
  }
  return fail("dq8_qlinear_f32: unknown epilogue");
}

namespace {

bool is_nhwc_ohwi(const int32_t md[17]) {
  static const int32_t want[12] = {0, 3, 1, 2, 3, 0, 1, 2, 0, 3, 1, 2};
  for (int i = 0; i < 12; ++i)
    if (md[i] != want[i]) return false;
  return true;
}

bool is_nchw_oihw(const int32_t md[17]) {
  static const int32_t want[12] = {0, 1, 2, 3, 1, 0, 2, 3, 0, 1, 2, 3};
  for (int i = 0; i < 12; ++i)
    if (md[i] != want[i]) return false;
  return true;
}

size_t pad256(int64_t v) { return (size_t)((v + 255) / 256 * 256); }

int out_elem_size(int epilogue) {
  return (epilogue == DQ8_EPI_ACC_S32 || epilogue == DQ8_EPI_DEQUANT_F32 ||
          epilogue == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 || epilogue == DQ8_EPI_REQUANT_GPU_DEQUANT_F32)
             ? 4 : 1;
}

int qconv2d_impl(int variant, const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                 const int64_t w_sizes[4], const int32_t padding[4], const int32_t md[17],
                 void* out, const int64_t out_sizes[4], int epilogue, const void* bias,
                 int bias_kind, const float* sx, const float* sw, int64_t n_sw, const float* so,
                 int32_t zo, void* workspace, size_t workspace_bytes, void* stream,
                 const dq8_postops_t* post = nullptr) {
  clear_error();
  DQ8_REQUIRE(in_sizes && w_sizes && padding && md && out_sizes, "dq8_qconv2d: null descriptor");
  DQ8_REQUIRE(variant >= -1 && variant < kNumVariants, "dq8_qconv2d: unknown variant");
  for (int i = 0; i < 12; ++i)
    DQ8_REQUIRE(md[i] >= 0 && md[i] < 4, "dq8_qconv2d: metadata dimension index out of range");
  for (int g = 0; g < 3; ++g) {
    int seen = 0;
    for (int i = 0; i < 4; ++i) seen |= 1 << md[4 * g + i];
    DQ8_REQUIRE(seen == 15, "dq8_qconv2d: metadata layout is not a permutation");
  }
  const int ib = md[0], ic = md[1], ih = md[2], iw = md[3];
  const int ki = md[4], ko = md[5], kh = md[6], kw = md[7];
  const int ob = md[8], oc = md[9], oh = md[10], ow = md[11];
  const int64_t NB = in_sizes[ib], H = in_sizes[ih], Wd = in_sizes[iw];
  int64_t Ci = in_sizes[ic];
  const int64_t Co = w_sizes[ko], Kh = w_sizes[kh], Kw = w_sizes[kw];
  const int64_t Ho = out_sizes[oh], Wo = out_sizes[ow];
  DQ8_REQUIRE(w_sizes[ki] == Ci, "dq8_qconv2d: kernel input features differ from the input's");
  DQ8_REQUIRE(out_sizes[ob] == NB && out_sizes[oc] == Co,
              "dq8_qconv2d: output batch/channel mismatch");
  const int sh = md[12], sw_ = md[13], dh = md[14], dw = md[15];
  DQ8_REQUIRE(sh > 0 && sw_ > 0 && dh > 0 && dw > 0, "dq8_qconv2d: strides/dilations must be > 0");
  DQ8_REQUIRE(padding[0] >= 0 && padding[1] >= 0 && padding[2] >= 0 && padding[3] >= 0,
              "dq8_qconv2d: negative padding");
  // the output extent must be what the geometry produces
  auto out_len = [](int64_t i, int64_t p0, int64_t p1, int64_t k, int64_t d, int64_t s) {
    return (i + p0 + p1 - k * d + d + s - 1) / s;
  };
  DQ8_REQUIRE(Ho == out_len(H, padding[0], padding[1], Kh, dh, sh) &&
                  Wo == out_len(Wd, padding[2], padding[3], Kw, dw, sw_),
              "dq8_qconv2d: output spatial size inconsistent with padding/stride/dilation");
  // Everything that can refuse the call is checked before any re-layout kernel is enqueued
  // (the re-layout branches below launch into the caller's scratch and then come back here
  // through a recursive call, which repeats these checks on its own arguments).
  {
    int ep = epilogue, rq = 0;
    if (ep == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 || ep == DQ8_EPI_REQUANT_GPU_DEQUANT_F32) {
      rq = 1;
      ep = ep == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 ? DQ8_EPI_REQUANT_CPU : DQ8_EPI_REQUANT_GPU;
    }
    if (ep == DQ8_EPI_REQUANT_FIXEDPOINT) {
      DQ8_REQUIRE(bias_kind == DQ8_BIAS_NONE || bias_kind == DQ8_BIAS_S32,
                  "dq8_qconv2d: the fixed-point stage takes an s32 bias or none");
      ep = DQ8_EPI_REQUANT_CPU;
    }
    if (int s = check_epilogue("dq8_qconv2d", ep, bias, bias_kind, sx, sw, so, 1, n_sw, 1, Co))
      return s;
    DQ8_REQUIRE(zo == 0 || ep == DQ8_EPI_REQUANT_CPU,
                "dq8_qconv2d: an output zero point needs the REQUANT_CPU epilogue");
    EpiParams dry = {};
    if (int s = apply_postops("dq8_qconv2d", post, !rq && elem_size(ep) == 1 && ep != DQ8_EPI_ACC_S32,
                              rq != 0, 1, Co, &dry))
      return s;
    DQ8_REQUIRE(!dry.resid_kind || is_nhwc_ohwi(md) || dry.ldr == Co,
                "dq8_qconv2d: a fused residual has the layout of the output");
  }

  // NCHW x OIHW -> NCHW (the PyTorch layouts): with scratch, the input and the weights are
  // re-laid out as NHWC / OHWI, the convolution runs on the MFMA kernels into an NHWC scratch
  // result, and that is turned back into NCHW -- what the reference's GPU path does around its
  // NHWC-only int8 kernels (R ral/context/stream_executor_based_impl.cc:1073-1112).  Without
  // scratch (or with a fused residual, which has the output's layout) the generic kernel reads
  // the tensors in place.
  if (is_nchw_oihw(md) && variant != 0 && workspace != nullptr && aligned(workspace, 256) &&
      !(post && post->residual_kind != DQ8_RESIDUAL_NONE) && NB <= 65535 && Co <= 65535 &&
      epilogue >= DQ8_EPI_ACC_S32 && epilogue <= DQ8_EPI_REQUANT_FIXEDPOINT) {
    const int64_t Mo = NB * out_sizes[2] * out_sizes[3];
    const int es = out_elem_size(epilogue);
    const size_t in_b = pad256(NB * H * Wd * Ci), w_b = pad256(Co * Kh * Kw * Ci);
    const size_t out_b = pad256(Mo * Co * es);
    if (workspace_bytes >= in_b + w_b + out_b && Mo > 0 && Co > 0 && in && w && out) {
      hipStream_t st0 = (hipStream_t)stream;
      int8_t* in_t = static_cast<int8_t*>(workspace);
      int8_t* w_t = in_t + in_b;
      uint8_t* out_t = reinterpret_cast<uint8_t*>(w_t + w_b);
      if (int s = transpose_batched<int8_t>(in, in_t, NB, Ci, H * Wd, st0)) return s;
      if (int s = transpose_batched<int8_t>(w, w_t, Co, Ci, Kh * Kw, st0)) return s;
      const int64_t in2[4] = {NB, H, Wd, Ci}, w2[4] = {Co, Kh, Kw, Ci};
      const int64_t out2[4] = {NB, out_sizes[2], out_sizes[3], Co};
      int32_t md2[17];
      static const int32_t nhwc[12] = {0, 3, 1, 2, 3, 0, 1, 2, 0, 3, 1, 2};
      for (int i = 0; i < 12; ++i) md2[i] = nhwc[i];
      for (int i = 12; i < 17; ++i) md2[i] = md[i];
      const size_t used = in_b + w_b + out_b;
      if (int s = qconv2d_impl(variant, in_t, in2, w_t, w2, padding, md2, out_t, out2, epilogue, bias,
                               bias_kind, sx, sw, n_sw, so, zo,
                               static_cast<uint8_t*>(workspace) + used, workspace_bytes - used,
                               stream, post))
        return s;
      const int64_t pix = out_sizes[2] * out_sizes[3];
      return es == 4 ? transpose_batched<uint32_t>(out_t, out, NB, pix, Co, st0)
                     : transpose_batched<int8_t>(out_t, out, NB, pix, Co, st0);
    }
  }

  // Stride 2 on an image of at most 4 channels (NHWC x OHWI, no dilation): with scratch, the
  // image goes through space to depth -- 2 x 2 pixels become the 16 channels of one, the
  // padding frame is written out -- and the weights likewise, and the convolution runs as a
  // ceil(K / 2)^2 stride-1 one on 16 channels.  Padding the 3 channels of a 7 x 7 stem to 16
  // instead costs 784 of k per output where this costs 256 (measured, batch 32 of 224 x 224:
  // 62-65 us that way).
  if (variant == -1 && is_nhwc_ohwi(md) && Ci >= 1 && Ci <= 4 && sh == 2 && sw_ == 2 &&
      dh == 1 && dw == 1 && workspace != nullptr && aligned(workspace, 256) && Ho > 0 && Wo > 0 &&
      NB > 0 && Co > 0 && NB + Co <= 65535 && Kh < (1 << 15) && Kw < (1 << 15) && in && w && out &&
      H < (1 << 15) && Wd < (1 << 15)) {
    const int64_t kbh = (Kh + 1) / 2, kbw = (Kw + 1) / 2;
    const int64_t Hb = Ho + kbh - 1, Wb = Wo + kbw - 1;
    const size_t in_b = pad256(NB * Hb * Wb * 16), w_b = pad256(Co * kbh * kbw * 16);
    if (workspace_bytes >= in_b + w_b) {
      hipStream_t st0 = (hipStream_t)stream;
      int8_t* in_t = static_cast<int8_t*>(workspace);
      int8_t* w_t = in_t + in_b;
      const SpaceToDepthJob job_in = {in, in_t, (int)NB, (int)H, (int)Wd, (int)Hb, (int)Wb, padding[0], padding[2]};
      const SpaceToDepthJob job_w = {w, w_t, (int)Co, (int)Kh, (int)Kw, (int)kbh, (int)kbw, 0, 0};
      if (int s = space_to_depth2_s8(job_in, job_w, (int)Ci, st0)) return s;
      const int64_t in2[4] = {NB, Hb, Wb, 16}, w2[4] = {Co, kbh, kbw, 16};
      const int32_t pad2[4] = {0, 0, 0, 0};
      int32_t md2[17];
      for (int i = 0; i < 17; ++i) md2[i] = md[i];
      md2[12] = md2[13] = 1;
      const size_t used = in_b + w_b;
      return qconv2d_impl(variant, in_t, in2, w_t, w2, pad2, md2, out, out_sizes, epilogue, bias,
                          bias_kind, sx, sw, n_sw, so, zo,
                          static_cast<uint8_t*>(workspace) + used, workspace_bytes - used, stream,
                          post);
    }
  }

  // requant -> dequantize in one epilogue, as in dq8_qgemm
  int requant = 0;
  if (epilogue == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 || epilogue == DQ8_EPI_REQUANT_GPU_DEQUANT_F32) {
    requant = epilogue == DQ8_EPI_REQUANT_CPU_DEQUANT_F32 ? 1 : 2;
    epilogue = requant == 1 ? DQ8_EPI_REQUANT_CPU : DQ8_EPI_REQUANT_GPU;
  }
  int fixedpoint = 0;
  if (epilogue == DQ8_EPI_REQUANT_FIXEDPOINT) {
    fixedpoint = 1;
    DQ8_REQUIRE(bias_kind == DQ8_BIAS_NONE || bias_kind == DQ8_BIAS_S32,
                "dq8_qconv2d: the fixed-point stage takes an s32 bias or none");
    epilogue = DQ8_EPI_REQUANT_CPU;
  }
  if (int s = check_epilogue("dq8_qconv2d", epilogue, bias, bias_kind, sx, sw, so, 1, n_sw, 1, Co))
    return s;
  DQ8_REQUIRE(zo == 0 || epilogue == DQ8_EPI_REQUANT_CPU,
              "dq8_qconv2d: an output zero point needs the REQUANT_CPU epilogue");
  if (requant) epilogue = DQ8_EPI_DEQUANT_F32;
  const int64_t Mg = NB * Ho * Wo;
  int64_t Kg = Kh * Kw * Ci;
  DQ8_REQUIRE(Mg < (1LL << 31) && Kg < (1LL << 31) && Co < (1LL << 31) &&
                  NB * H * Wd * Ci < (1LL << 40),
              "dq8_qconv2d: problem too large");
  if (Mg == 0 || Co == 0) return 0;
  DQ8_REQUIRE(in && w && out, "dq8_qconv2d: null tensor");
  hipStream_t st = (hipStream_t)stream;

  EpiParams e = {};
  e.out = out;
  e.ldo = Co;
  e.M = (int)Mg;
  e.N = (int)Co;
  e.bias = bias;
  e.bias_kind = bias_kind;
  e.sx = sx;
  e.sw = sw;
  e.so = so;
  e.sx_stride = 0;
  e.sw_stride = n_sw > 1;
  e.so_stride = 0;
  e.zo = zo;
  e.requant = requant;
  e.fixedpoint = fixedpoint;
  const int es = elem_size(epilogue);
  e.vec_store = aligned(out, 4 * es) && (Co % 4 == 0);
  e.vec_store16 = aligned(out, 16) && (Co % 16 == 0);
  if (int s = apply_postops("dq8_qconv2d", post, es == 1 && epilogue != DQ8_EPI_ACC_S32,
                            requant != 0, 1, Co, &e))
    return s;
  DQ8_REQUIRE(!e.resid_kind || is_nhwc_ohwi(md) || e.ldr == Co,
              "dq8_qconv2d: a fused residual has the layout of the output");

  const bool nhwc_ohwi = is_nhwc_ohwi(md);
  const bool auto_pick = variant == -1;
  // Channel counts that are not a multiple of 16 (an RGB first layer): with scratch, input
  // and weights are rewritten with the channels zero-filled up to the next multiple; the
  // added channels contribute nothing and the MFMA kernels run on the padded tensors.
  // (fused operators with an output the 16-byte stores cannot take run on the generic kernel,
  // which reads the tensors as they were passed)
  const bool fused = e.table != nullptr || e.resid_kind != 0;
  const bool fused_ok = !fused || (es == 1 ? e.vec_store16 : e.vec_store);
  const int64_t Cip = (Ci + 15) / 16 * 16;
  if (nhwc_ohwi && Ci % 16 != 0 && variant != 0 && fused_ok && workspace != nullptr &&
      aligned(workspace, 256) &&
      workspace_bytes >= pad256(NB * H * Wd * Cip) + pad256(Co * Kh * Kw * Cip) &&
      NB * H * Wd * Cip < (1LL << 40) && Kh * Kw * Cip < (1LL << 31)) {
    int8_t* in_p = (int8_t*)workspace;
    int8_t* w_p = in_p + pad256(NB * H * Wd * Cip);
    auto blocks = [](int64_t rows, int64_t ldd) {
      return dim3((unsigned)std::min<int64_t>(ceil_div(rows * (ldd / 16), 256), 1 << 20));
    };
    hipLaunchKernelGGL(pad_rows_s8_kernel, blocks(NB * H * Wd, Cip), dim3(256), 0, st, in, Ci,
                       in_p, NB * H * Wd, (int)Ci, (int)Cip);
    hipLaunchKernelGGL(pad_rows_s8_kernel, blocks(Co * Kh * Kw, Cip), dim3(256), 0, st, w, Ci,
                       w_p, Co * Kh * Kw, (int)Ci, (int)Cip);
    DQ8_HIP(hipGetLastError());
    in = in_p;
    w = w_p;
    Ci = Cip;
    Kg = Kh * Kw * Ci;
  }
  const bool fast_ok = nhwc_ohwi && Ci % 16 == 0 && aligned(in, 16) && aligned(w, 16) && fused_ok;
  if (auto_pick && !fast_ok) variant = 0;
  if (variant != 0)
    DQ8_REQUIRE(fast_ok, "dq8_qconv2d: the MFMA variants need NHWC x OHWI, Ci % 16 == 0 and "
                         "16-byte aligned tensors");
  if (variant == 0) {
    auto strides = [](const int64_t s[4], int64_t st4[4]) {
      st4[3] = 1;
      for (int i = 3; i > 0; --i) st4[i - 1] = st4[i] * s[i];
    };
    int64_t is[4], ws[4], os[4];
    strides(in_sizes, is);
    strides(w_sizes, ws);
    strides(out_sizes, os);
    GenericConvParams g;
    g.in = in;
    g.w = w;
    g.i_sb = is[ib]; g.i_sc = is[ic]; g.i_sh = is[ih]; g.i_sw = is[iw];
    g.w_si = ws[ki]; g.w_so = ws[ko]; g.w_sh = ws[kh]; g.w_sw = ws[kw];
    g.o_sb = os[ob]; g.o_sc = os[oc]; g.o_sh = os[oh]; g.o_sw = os[ow];
    g.NB = (int)NB; g.H = (int)H; g.Wd = (int)Wd; g.Ci = (int)Ci; g.Co = (int)Co;
    g.Kh = (int)Kh; g.Kw = (int)Kw; g.Ho = (int)Ho; g.Wo = (int)Wo;
    g.pad_t = padding[0]; g.pad_l = padding[2];
    g.sh = sh; g.sw_ = sw_; g.dh = dh; g.dw = dw;
    g.epi = e;
    return launch_generic_epi<GenericConvParams>(
        qconv_generic_kernel<DQ8_EPI_ACC_S32>, qconv_generic_kernel<DQ8_EPI_REQUANT_CPU>,
        qconv_generic_kernel<DQ8_EPI_REQUANT_GPU>, qconv_generic_kernel<DQ8_EPI_DEQUANT_F32>,
        epilogue, g, Mg * Co, st);
  }

  // A 1x1 filter with stride 1 and no padding is a plain GEMM over the pixels.
  const bool pointwise = Kh == 1 && Kw == 1 && sh == 1 && sw_ == 1 && padding[0] == 0 &&
                         padding[1] == 0 && padding[2] == 0 && padding[3] == 0;
  // what the streaming kernel asks of the output side
  const bool stream_out = !e.fixedpoint && e.vec_store16 &&
                          (epilogue == DQ8_EPI_REQUANT_CPU || epilogue == DQ8_EPI_REQUANT_GPU);
  // On 64 to 256 input channels the filter fits the registers of the streaming kernel; its
  // pixels are then one long row, cut into patch rows of 16 where the count allows, so that a
  // tile is any run of pixels, across images.
  if (pointwise && (auto_pick || variant == kStreamConv)) {
    DirectConvParams sp = {};
    sp.in = in;
    sp.w = w;
    sp.Ci = (int)Ci; sp.Co = (int)Co;
    sp.Kh = 1; sp.Kw = 1;
    if (Mg % 16 == 0 && Mg / 16 < (1LL << 24)) {
      sp.NB = 1; sp.H = sp.Ho = (int)(Mg / 16); sp.Wd = sp.Wo = 16;
    } else {
      sp.NB = (int)NB; sp.H = sp.Ho = (int)Ho; sp.Wd = sp.Wo = (int)Wo;
    }
    sp.epi = e;
    const bool ok = stream_out && Ci <= 256 && (Ci <= 128 || !fused) && stream_conv_has_instance(1, 1, (int)Ci) &&
                    stream_conv_plan(&sp);
    if (!auto_pick)
      DQ8_REQUIRE(ok, "dq8_qconv2d: the streaming variant needs a 3 x 3 or 1 x 1 filter on 64 or "
                      "128 input channels (1 x 1 without fused operators also on 256), stride and "
                      "dilation 1, an int8 result (float output stage) and 16-byte aligned output "
                      "rows");
    // Against the GEMM kernels, whose k tile of 128 is half empty at 64 channels and whose
    // workgroups requantise in lock step, it wins once the launch has a few million results
    // (us per launch, streaming / GEMM; 64 -> 256 channels on 56 x 56 images: batch 1 4.1 / 3.5,
    // batch 4 4.7 / 4.7, batch 8 5.45 / 7.6, batch 32 11.2 / 15.3, batch 64 17.6 / 26.3; 64 -> 64,
    // batch 32: 28 x 28 3.7 / 4.5, 56 x 56 5.5 / 7.0, 112 x 112 12.7 / 19.3; 128 -> 128, batch 32:
    // 28 x 28 5.0 / 4.7, 56 x 56 8.7 / 12.1; 128 -> 256 on 28 x 28: 5.8 / 7.7; 128 -> 512: 8.6 / 8.8,
    // batch 64 12.6 / 15.4).
    // 256 channels (64-channel slices; every slice of a pixel tile loads the tile's pixels again):
    // while the workgroups are one round of the chip or the slices are at most two -- 32 x 14 x 14
    // x 256 -> 1024 5.5 / 6.55, 32 x 56 x 56 x 256 -> 64 6.4 / 7.65, -> 128 10.3 / 11.5, 32 x 28 x 28
    // x 256 -> 256 5.7 / 6.7; several rounds of many slices lose: 64 x 28 x 28 x 256 -> 256
    // 9.9 / 8.8, 32 x 56 x 56 x 256 -> 512 31.1 / 28.4; below 1.5 M results the GEMM tiles are
    // as fast (4 x 14 x 14 x 256 -> 1024 3.85 / 3.8).
    const bool take = Ci == 64    ? Mg * Co >= (3LL << 19)
                      : Ci == 128 ? Mg * Co >= (6LL << 20)
                                  : Mg * Co >= (3LL << 19) &&
                                        (Co <= 128 || (int64_t)sp.NB * sp.tiles_per_image * sp.tiles_n <=
                                                          compute_units());
    if (ok && (!auto_pick || take))
      return launch_stream_conv(epilogue, sp, st);
  }
  // Otherwise the GEMM instantiations load its rows without the per-tap address arithmetic.
  if (auto_pick && pointwise) {
    MainParams g = {};
    g.A = in;
    g.W = w;
    g.lda = Ci;
    g.ldw = Ci;
    g.M = (int)Mg;
    g.N = (int)Co;
    g.K = (int)Ci;
    g.epi = e;
    int v = pick_any(Mg, Co, Ci, pipe_ok(256, 256, g, false), es);
    if (fused || e.fixedpoint) {   // the persistent forms carry neither
      if (v == kPersist256) v = kPipe256w8;
      if (v == kPersist256x192) v = kPipe256x192;
      if (v == kPersist128) v = kPipe128w8;
    }
    return launch_epi<false>(v, g, epilogue, st);
  }

  // A 1 x 1 filter with a stride and no padding is the same GEMM over the pixels it reads: the
  // one-tile pipelined kernels find a row's pixel once, before their k loop, and run the plain
  // GEMM's loop without the per-tap address arithmetic (stride 2, batch 32, against the best
  // implicit-GEMM tile: 56 x 56 x 256 -> 512 10.3 -> 9.7 us, 28 x 28 x 512 -> 1024 9.9 -> 9.15,
  // 14 x 14 x 1024 -> 2048 8.95 -> 7.8; batch 8: 5.9 -> 5.3, 6.3 -> 5.7, 6.7 -> 5.7).
  if (auto_pick && Kh == 1 && Kw == 1 && !pointwise && padding[0] == 0 && padding[1] == 0 &&
      padding[2] == 0 && padding[3] == 0 && NB * H * Wd * Ci < (1LL << 31)) {
    MainParams g = {};
    g.A = in;
    g.W = w;
    g.lda = Ci;
    g.ldw = Ci;
    g.M = (int)Mg;
    g.N = (int)Co;
    g.K = (int)Ci;
    g.H = (int)H; g.Wd = (int)Wd; g.Ci = (int)Ci; g.Ho = (int)Ho; g.Wo = (int)Wo;
    g.sh = sh; g.sw_ = sw_;
    g.conv_bytes = NB * H * Wd * Ci;
    g.epi = e;
    int v = pick_any(Mg, Co, Ci, pipe_ok(256, 256, g, false), es);
    if (v == kPersist256) v = kPipe256w8;
    if (v == kPersist256x192) v = kPipe256x192;
    if (v == kPersist128) v = kPipe128w8;
    if (rowmap_has_variant(v) && pipe_ok(kVariants[v].bm, kVariants[v].bn, g, false))
      return launch_rowmap_epi(v, g, epilogue, st);
  }

  MainParams p = {};
  p.A = in;
  p.W = w;
  p.lda = 0;
  p.ldw = Kg;
  p.M = (int)Mg;
  p.N = (int)Co;
  p.K = (int)Kg;
  p.H = (int)H; p.Wd = (int)Wd; p.Ci = (int)Ci; p.Ho = (int)Ho; p.Wo = (int)Wo;
  p.Kh = (int)Kh; p.Kw = (int)Kw;
  p.pad_t = padding[0]; p.pad_l = padding[2];
  p.sh = sh; p.sw_ = sw_; p.dh = dh; p.dw = dw;
  p.conv_bytes = NB * H * Wd * Ci;
  p.epi = e;

  DirectConvParams d = {};
  d.in = in;
  d.w = w;
  d.NB = (int)NB; d.H = (int)H; d.Wd = (int)Wd; d.Ci = (int)Ci; d.Co = (int)Co;
  d.Ho = (int)Ho; d.Wo = (int)Wo;
  d.pad_t = padding[0]; d.pad_l = padding[2];
  d.Kh = (int)(Kh < 64 ? Kh : 64); d.Kw = (int)(Kw < 64 ? Kw : 64);
  d.epi = e;
  // (3 x 3 in the first place; any filter up to 7 x 7 with more than one tap runs the same way)
  const bool direct_shape = Kh * Kw > 1 && Kh <= 7 && Kw <= 7 && sh == 1 && sw_ == 1 && dh == 1 &&
                            dw == 1 && padding[0] < Kh && padding[2] < Kw;
  if ((variant >= kDirectConv0 && variant < kDirectConv0 + 2) || variant == kDirectConv2) {
    const int config = variant == kDirectConv2 ? 2 : variant - kDirectConv0;
    DQ8_REQUIRE(direct_shape && direct_conv_plan(config, &d),
                "dq8_qconv2d: the direct variants need a filter of 2 to 7 x 7 taps with stride and "
                "dilation 1, Ci in {32, 64, 128, 256} (or 16 with an even filter width) and a "
                "patch that fits the LDS");
    return launch_direct_conv(config, epilogue, d, st);
  }
  // 3 x 3 filters on 64 or 128 channels with int8 results: the filter in registers
  const bool stream_shape = direct_shape && Ci <= 128 && stream_conv_has_instance((int)d.Kh, (int)d.Kw, (int)Ci) &&
                            stream_out;
  if (variant == kStreamConv) {
    DQ8_REQUIRE(stream_shape && stream_conv_plan(&d),
                "dq8_qconv2d: the streaming variant needs a 3 x 3 or 1 x 1 filter on 64 or "
                "128 input channels (or 4 x 4 on 16), stride and dilation 1, an int8 result "
                "(float output stage) and 16-byte aligned output rows");
    return launch_stream_conv(epilogue, d, st);
  }
  if (auto_pick) {
    // The streaming kernel wins at every size on 64 input channels (batch 1 to 128 of
    // 56 x 56 x 64 -> 64: 4.9-22.1 us against 6.3-32.7 for the best of the other kernels); on 128
    // channels, where a pixel tile's patch is loaded by four 32-channel slices, while the
    // workgroups are one round of the chip (32 x 28 x 28 x 128 -> 128: 8.3 against 9.3 us; batch
    // 8: 5.1 / 6.7; batch 64, two rounds: 14.7 against 14.3 for the 128 x 128 tiles).
    if (stream_shape) {
      DirectConvParams sp = d;
      if (stream_conv_plan(&sp) &&
          (Ci <= 64 || (int64_t)sp.NB * sp.tiles_per_image * sp.tiles_n <= compute_units()))
        return launch_stream_conv(epilogue, sp, st);
    }
    if (direct_shape) {
      const int c = pick_direct_conv(NB, Ho * Wo, Ci, Co);
      if (c >= 0 && direct_conv_plan(c, &d)) return launch_direct_conv(c, epilogue, d, st);
    }
    variant = pick_variant(Mg, Co, Kg, pipe_ok(256, 256, p, true), es);
    // (the persistent forms are tuned for the plain GEMM: with the convolution's row geometry
    // on top they run out of registers)
    if (variant == kPersist256) variant = kPipe256w8;
    if (variant == kPersist256x192) variant = kPipe256x192;
    if (variant == kPersist128) variant = kPipe128w8;
    // As implicit GEMMs the 256-row tiles, which the estimate takes from two rounds of 128 x 128
    // tiles on, lose to the four-wave 128 x 128 tile where half their columns are empty (up to
    // 128 output channels) or where they do not fill three quarters of the compute units (3 x 3
    // x 128 filters: 64 x 28 x 28 -> 128 14.3 against 16.3 us, 128 x 28 x 28 27.1 / 31.8,
    // 32 x 56 x 56 27.3 / 32.0, 32 x 28 x 28 -> 256 15.4 / 17.0; 64 x 28 x 28 x 256 -> 256, 196
    // tiles of 256 x 256, keeps them: 33.7 against 44.5 us).
    if ((variant == kPipe256w8 || variant == kPipe256x192) && pipe_ok(128, 128, p, true) &&
        (Co <= 128 || (Co <= 256 && 4 * ceil_div(Mg, 256) * ceil_div(Co, 256) < 3 * compute_units())))
      // (eight waves while the 128 x 128 tiles are at most one per compute unit, as for the
      // plain GEMM: 32 x 56 x 56 x 128 -> 128, 3 x 3 stride 2, 196 tiles: 8.9 against 9.7 us)
      variant = es == 1 && ceil_div(Mg, 128) * ceil_div(Co, 128) <= compute_units() ? kPipe128w8 : kPipe128;
  }
  return launch_epi<true>(variant, p, epilogue, st);
}

}  // namespace

extern "C" size_t dq8_qconv2d_workspace_bytes_ex(const int64_t in_sizes[4],
                                                 const int64_t w_sizes[4],
                                                 const int64_t out_sizes[4],
                                                 const int32_t metadata[17]) {
  if (!in_sizes || !w_sizes || !metadata) return 0;
  if (is_nchw_oihw(metadata)) {
    // NHWC copies of input and weights, an NHWC result of up to 4 bytes per element, and what
    // the NHWC convolution may want for itself
    if (!out_sizes) return 0;
    const int64_t ci = in_sizes[1], cip = (ci + 15) / 16 * 16;
    const int64_t in_e = in_sizes[0] * in_sizes[2] * in_sizes[3];
    const int64_t w_e = w_sizes[0] * w_sizes[2] * w_sizes[3];
    size_t need = pad256(in_e * ci) + pad256(w_e * ci) +
                  pad256(out_sizes[0] * out_sizes[1] * out_sizes[2] * out_sizes[3] * 4);
    if (ci % 16 != 0) need += pad256(in_e * cip) + pad256(w_e * cip);
    return need;
  }
  if (!is_nhwc_ohwi(metadata)) return 0;
  const int64_t ci = in_sizes[3];
  if (ci % 16 == 0) return 0;
  const int64_t cip = (ci + 15) / 16 * 16;
  size_t need = pad256(in_sizes[0] * in_sizes[1] * in_sizes[2] * cip) +
                pad256(w_sizes[0] * w_sizes[1] * w_sizes[2] * cip);
  // (the space-to-depth copies of a stride-2 convolution with at most 4 channels; smaller
  // than the padded copies except for images of a few pixels)
  if (ci <= 4 && out_sizes && metadata[12] == 2 && metadata[13] == 2) {
    const int64_t kbh = (w_sizes[1] + 1) / 2, kbw = (w_sizes[2] + 1) / 2;
    const size_t s2d = pad256(in_sizes[0] * (out_sizes[1] + kbh - 1) * (out_sizes[2] + kbw - 1) * 16) +
                       pad256(w_sizes[0] * kbh * kbw * 16);
    if (s2d > need) need = s2d;
  }
  return need;
}

extern "C" size_t dq8_qconv2d_workspace_bytes(const int64_t in_sizes[4], const int64_t w_sizes[4],
                                              const int32_t metadata[17]) {
  return dq8_qconv2d_workspace_bytes_ex(in_sizes, w_sizes, nullptr, metadata);
}

#ifdef DQ8_TEST_HOOKS
extern "C" int dq8_qconv2d_variant(int variant, const int8_t* in, const int64_t in_sizes[4],
                                   const int8_t* w, const int64_t w_sizes[4],
                                   const int32_t padding[4], const int32_t md[17],
                                   void* out, const int64_t out_sizes[4], int epilogue,
                                   const void* bias, int bias_kind, const float* sx,
                                   const float* sw, int64_t n_sw, const float* so,
                                   int32_t zo, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  return qconv2d_impl(variant, in, in_sizes, w, w_sizes, padding, md, out, out_sizes, epilogue,
                      bias, bias_kind, sx, sw, n_sw, so, zo, workspace, workspace_bytes, stream);
}
#endif

extern "C" int dq8_qconv2d_ws(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                              const int64_t w_sizes[4], const int32_t padding[4],
                              const int32_t metadata[17], void* out, const int64_t out_sizes[4],
                              int epilogue, const void* bias, int bias_kind, const float* sx,
                              const float* sw, int64_t n_sw, const float* so, int32_t zo,
                              void* workspace, size_t workspace_bytes, void* stream) {
  return qconv2d_impl(-1, in, in_sizes, w, w_sizes, padding, metadata, out, out_sizes, epilogue,
                      bias, bias_kind, sx, sw, n_sw, so, zo, workspace, workspace_bytes, stream);
}

extern "C" int dq8_qconv2d_fused(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                                 const int64_t w_sizes[4], const int32_t padding[4],
                                 const int32_t metadata[17], void* out,
                                 const int64_t out_sizes[4], int epilogue, const void* bias,
                                 int bias_kind, const float* sx, const float* sw, int64_t n_sw,
                                 const float* so, int32_t zo, void* workspace,
                                 size_t workspace_bytes, const dq8_postops_t* post, void* stream) {
  return qconv2d_impl(-1, in, in_sizes, w, w_sizes, padding, metadata, out, out_sizes, epilogue,
                      bias, bias_kind, sx, sw, n_sw, so, zo, workspace, workspace_bytes, stream,
                      post);
}

extern "C" int dq8_qconv2d(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                           const int64_t w_sizes[4], const int32_t padding[4],
                           const int32_t metadata[17], void* out, const int64_t out_sizes[4],
                           int epilogue, const void* bias, int bias_kind, const float* sx,
                           const float* sw, int64_t n_sw, const float* so, int32_t zo,
                           void* stream) {
  return qconv2d_impl(-1, in, in_sizes, w, w_sizes, padding, metadata, out, out_sizes, epilogue,
                      bias, bias_kind, sx, sw, n_sw, so, zo, nullptr, 0, stream);
}

#ifdef DQ8_TEST_HOOKS
extern "C" int dq8_mfma_probe(const int8_t* a, const int8_t* b, int32_t* d32,
                              const int8_t* a16, const int8_t* b16, int32_t* d16,
                              void* stream) {
  clear_error();
  DQ8_REQUIRE(a && b && d32 && a16 && b16 && d16, "dq8_mfma_probe: null pointer");
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, a, b, d32,
                     a16, b16, d16);
  return check_hip(hipGetLastError(), "dq8_mfma_probe launch");
}
#endif
