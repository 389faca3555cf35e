// Host launchers of the tiled int8 GEMM / implicit-GEMM convolution kernels: the table of tile
// variants and launch_variant<CONV, EPI>, which instantiates every kernel of one (operation,
// epilogue) pair.  Each pair is compiled in a translation unit of its own (qgemm_launch_*.hip),
// so that the kernels build in parallel; qgemm.hip only declares them.
#ifndef DQ8_QGEMM_LAUNCH_H_
#define DQ8_QGEMM_LAUNCH_H_

#include <cstdlib>

#include "dq8_common.h"
#include "disc_q8.h"
#include "qgemm_device.h"
#include "qgemm_pipelined.h"
#include "qgemm_persistent.h"
#include "qgemm_skinny.h"

#pragma clang fp contract(off)

namespace dq8 {

// ------------------------------------------------------------- tile variants
struct Variant {
  const char* name;
  int bm, bn, bk, threads;
};
// index 0 is the generic scalar kernel
inline constexpr Variant kVariants[] = {
    {"generic", 1, 1, 1, 256},
    {"mfma_256x256x64_w2x2", 256, 256, 64, 256},
    {"mfma_128x128x64_w2x2", 128, 128, 64, 256},
    {"mfma_64x64x64_w2x2", 64, 64, 64, 256},
    // software-pipelined kernels, operands loaded straight into LDS (the 256 x 256 tile on four
    // waves -- here and in the basic kernel above -- keeps 256 accumulators per lane and spills
    // part of their indexing: superseded by the eight-wave form, kept as a cross-check variant
    // that the library never picks by itself)
    {"pipe_256x256x128", 256, 256, 128, 256},
    {"pipe_128x128x128", 128, 128, 128, 256},
    {"pipe_64x64x128", 64, 64, 128, 256},
    {"pipe_256x64x128", 256, 64, 128, 256},
    // the same with the k tiles split over 2 groups of waves inside the workgroup
    {"pipe_64x64x128_k2", 64, 64, 128, 512},
    // small-M kernel: 16 output channels per workgroup, K split over the waves (GEMM only)
    {"skinny_16", 16, 16, 64, 512},
    // 3x3 stride-1 convolution with the input patch resident in LDS (convolution only)
    {"direct3x3_256x64", 256, 64, 128, 256},
    {"direct3x3_128x64", 128, 64, 128, 256},
    // eight waves per workgroup: 256x256 with wave tile 128x64 (two waves per SIMD), 128x128
    // with wave tile 64x32 (two workgroups per CU: four waves per SIMD)
    {"pipe_256x256x128_w8", 256, 256, 128, 512},
    {"pipe_128x128x128_w8", 128, 128, 128, 512},
    // persistent forms: one workgroup per slot walks several tiles, the next tile's first
    // loads fly during the epilogue
    {"persist_256x256x128_w8", 256, 256, 128, 512},
    {"persist_128x128x128_w8", 128, 128, 128, 512},
    // 256x192 on eight waves (wave tile 64x96): for problems whose 256x256 tiles would leave
    // a quarter of the compute units idle
    {"pipe_256x192x128_w8", 256, 192, 128, 512},
    {"persist_256x192x128_w8", 256, 192, 128, 512},
    // the third direct-convolution tile: 512 pixels on eight waves, one workgroup per compute
    // unit (convolution only)
    {"direct3x3_512x64", 512, 64, 128, 512},
    // 64x64 with the k tiles split over 4 groups of waves (sixteen waves, 128 KiB LDS)
    {"pipe_64x64x128_k4", 64, 64, 128, 1024},
    // a filter slice held in registers (3 x 3 or 1 x 1 on 64 or 128 channels), pixel tile chosen
    // per problem (convolution only, int8 results)
    {"stream", 32, 64, 32, 512},
};
constexpr int kPipe256 = 4, kPipe128 = 5, kPipe64 = 6, kPipe256x64 = 7;
constexpr int kPipe64k2 = 8;
constexpr int kSkinnyVariant = 9;
constexpr int kDirectConv0 = 10;   // first of the kNumDirectConvConfigs direct variants
constexpr int kPipe256w8 = 12, kPipe128w8 = 13;
constexpr int kPersist256 = 14, kPersist128 = 15;
constexpr int kPipe256x192 = 16, kPersist256x192 = 17;
constexpr int kDirectConv2 = 18;   // the third direct variant (configuration 2)
constexpr int kPipe64k4 = 19;
constexpr int kStreamConv = 20;
// largest M the heuristic hands to the small-M kernel
constexpr int64_t kSkinnyMaxM = 32;
// Above that many rows the small-M kernel still beats the 64 x 64 tiles while its workgroups
// (16 rows x 16 channels, each over all of k) are few: up to 256 rows and
// ceil(M / 16) ceil(N / 16) ceil(K / 768) <= 1024, or 3072 from 2048 of k on, where the tiles'
// k loop is long (us per launch, small-M kernel against tiles: M = 64, 768 -> 768: 3.2 / 4.8;
// M = 256: 4.1 / 4.7; M = 64, 768 -> 3072: 4.1 / 4.6; M = 128: 5.1 / 4.9; M = 64, 3072 -> 768:
// 4.3 / 7.7; M = 256: 6.5 / 7.8; M = 64, 4096^2: 8.7 / 9.2; M = 128: 13.6 / 9.2).
inline bool skinny_takes_rows(int64_t M, int64_t N, int64_t K) {
  if (M <= kSkinnyMaxM) return true;
  if (M > 256) return false;
  const int64_t units = ceil_div(M, 16) * ceil_div(N, 16) * ceil_div(K, 768);
  return units <= (K >= 2048 ? 3072 : 1024);
}

inline bool is_pipe_variant(int v) {
  return v == kPipe256 || v == kPipe128 || v == kPipe64 || v == kPipe256x64 || v == kPipe64k2 ||
         v == kPipe64k4 || v == kPipe256w8 || v == kPipe128w8 || v == kPersist256 ||
         v == kPersist128 || v == kPipe256x192 || v == kPersist256x192;
}
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);


template <int BM, int BN, int BK, int WM, int WN, bool CONV, int EPI>
int launch_mfma(const MainParams& p, hipStream_t st) {
  constexpr int lds = 2 * (BM + BN) * (BK + 16);
  auto kern = qgemm_mfma_kernel<BM, BN, BK, WM, WN, CONV, EPI>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds, &lds_allowed)) return s;
  const int grid = p.tiles_m * p.tiles_n;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(WM * WN * 64), lds, st, p);
  return check_hip(hipGetLastError(), "qgemm_mfma launch");
}

// The pipelined kernels address each block's rows (GEMM) or the whole image
// (convolution) with 32-bit buffer offsets.
inline bool pipe_ok(int bm, int bn, const MainParams& p, bool conv) {
  constexpr int BK = 128;
  if (p.K < 16 || p.K % 16 != 0) return false;
  if ((int64_t)bn * p.ldw + p.K + 2 * BK >= (1LL << 31)) return false;
  if (conv) return p.conv_bytes < (1LL << 31) && p.Ci % 16 == 0;
  return (int64_t)bm * p.lda + p.K + 2 * BK < (1LL << 31);
}

template <int BM, int BN, int WM, int WN, int KSPLIT, bool CONV, int EPI, bool ROWMAP = false>
int launch_pipe(const MainParams& p, hipStream_t st) {
  constexpr int BK = 128;
  constexpr int lds = KSPLIT * 2 * (BM + BN) * BK;
  DQ8_REQUIRE(pipe_ok(BM, BN, p, CONV) && (!ROWMAP || p.conv_bytes < (1LL << 31)),
              "pipelined qgemm needs K % 16 == 0 and operands that fit 32-bit buffer offsets");
  auto kern = qgemm_pipe_kernel<BM, BN, WM, WN, KSPLIT, CONV, EPI, ROWMAP>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds, &lds_allowed)) return s;
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(WM * WN * KSPLIT * 64), lds, st, p);
  return check_hip(hipGetLastError(), "qgemm_pipe launch");
}

// `per_cu`: workgroups of this shape a compute unit holds at a time
template <int BM, int BN, int WM, int WN, bool CONV, int EPI>
int launch_persist(const MainParams& p, int per_cu, hipStream_t st) {
  constexpr int stage = (BM + BN) * 128;
  // (per-channel factors: 8 bytes, plus 4 for the shifts of the fixed-point output stage, and
  // the 256-byte table of a fused lookup)
  constexpr int lds = 2 * stage + (WM * WN * 4096 + BN * 12 + 256 <= stage ? 0 : BN * 12 + 256);
  DQ8_REQUIRE(pipe_ok(BM, BN, p, CONV),
              "persistent qgemm needs K % 16 == 0 and operands that fit 32-bit buffer offsets");
  auto kern = qgemm_persist_kernel<BM, BN, WM, WN, CONV, EPI>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds, &lds_allowed)) return s;
  const int tiles = p.tiles_m * p.tiles_n;
  const int slots = compute_units() * per_cu;
  hipLaunchKernelGGL(kern, dim3(tiles < slots ? tiles : slots), dim3(WM * WN * 64), lds, st, p);
  return check_hip(hipGetLastError(), "qgemm_persist launch");
}

template <int NW, int MT, int EPI, int U = 4>
int launch_skinny_t(const MainParams& p, hipStream_t st) {
  const dim3 grid((unsigned)ceil_div(p.N, 16), (unsigned)ceil_div(p.M, 16 * MT));
  DQ8_REQUIRE(grid.y <= 65535, "small-M qgemm: M too large for this variant");
  hipLaunchKernelGGL((qgemm_skinny_kernel<NW, MT, EPI, U>), grid, dim3(NW * 64), 0, st, p);
  return check_hip(hipGetLastError(), "qgemm_skinny launch");
}

template <int MR, int U, int EPI>
int launch_gemv_t(const MainParams& p, hipStream_t st) {
  auto kern = qgemm_gemv_kernel<8, MR, U, EPI>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, &lds_allowed)) return s;
  hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(p.N, 8)), dim3(512), MR * p.K, st, p);
  return check_hip(hipGetLastError(), "qgemm_gemv launch");
}

// rows per workgroup grow with M (fewer passes over W), waves with the depth of K
template <int EPI>
int launch_skinny(const MainParams& p, hipStream_t st) {
  // one or two rows against rows of at least 2048 of k (two steps of a wave): the
  // row-streaming kernel (M = 1, 3072 -> 768: 3.1 against 4.0 us; 4096^2: 3.8 against 5.0;
  // 8192^2: 12.7 against 14.2 us, 5.3 TB/s; at 768 of k, and from three rows on, it is slower)
  if (p.M <= 2 && p.K >= 2048 && (int64_t)2 * p.K <= 64 * 1024) {
    const bool deep8 = p.K > 4096;
    if (p.M == 1) return deep8 ? launch_gemv_t<1, 8, EPI>(p, st) : launch_gemv_t<1, 4, EPI>(p, st);
    return deep8 ? launch_gemv_t<2, 8, EPI>(p, st) : launch_gemv_t<2, 4, EPI>(p, st);
  }
  // Waves: four, eight from 1024 of k on (M = 16, 3072 -> 768: 4.1 against 4.3 us).  Row tiles
  // of 16 per workgroup: one, i.e. as many workgroups as possible, while the weights, which
  // every block of rows streams again, stay below about 20 MB over all its passes; else two or
  // four (us per launch, graph replays, for (waves, row tiles) = (4,1) (4,2) (4,4) / (8,1) (8,2)
  // (8,4): M = 64, 768 -> 768: 3.2 3.9 4.9; M = 256, 768 -> 3072: 7.3 7.0 7.5; M = 32, 4096^2:
  // 7.2 6.3 7.3 (eight waves); M = 64, 4096^2: 10.7 9.4 8.7; M = 128, 3072 -> 768: 5.7 5.0 6.8).
  const bool deep = p.K >= 1024;
  const int64_t weight_bytes = (int64_t)p.N * p.K;
  int mt = 1;
  while (mt < 4 && ceil_div(p.M, 16 * mt) * weight_bytes > (20LL << 20)) mt *= 2;
  // k-steps a wave keeps in flight: as many as it has altogether up to six -- a batch that is
  // not full still issues all its loads (3072 of k on eight waves, six steps each: 4.1 -> 3.8 us
  // at M = 16, 7.5 -> 6.9 at M = 256; 768 of k on four waves, three steps: M = 128, -> 3072 5.4 ->
  // 4.9 us; 1024 of k on eight, two steps: 3.5 -> 3.15 us) -- and four from seven steps on
  // unless batches of six leave fewer idle slots.
  const int64_t steps = ceil_div(ceil_div(p.K, 64), deep ? 8 : 4);
  int u = 4;
  if (steps <= 2) u = 2;
  else if (steps == 3) u = 3;
  else if (steps == 5 || steps == 6) u = 6;
  else if (steps >= 7 && deep && ceil_div(steps, 6) * 6 < ceil_div(steps, 4) * 4) u = 6;
  if (mt <= 2) {
#define DQ8_SKINNY_CASE(NW_, U_)                                              \
  if (u == U_) return mt == 1 ? launch_skinny_t<NW_, 1, EPI, U_>(p, st)      \
                              : launch_skinny_t<NW_, 2, EPI, U_>(p, st);
    if (deep) {
      DQ8_SKINNY_CASE(8, 2) DQ8_SKINNY_CASE(8, 3) DQ8_SKINNY_CASE(8, 6) DQ8_SKINNY_CASE(8, 4)
    } else {
      DQ8_SKINNY_CASE(4, 2) DQ8_SKINNY_CASE(4, 3) DQ8_SKINNY_CASE(4, 4)
      return mt == 1 ? launch_skinny_t<4, 1, EPI, 4>(p, st) : launch_skinny_t<4, 2, EPI, 4>(p, st);
    }
#undef DQ8_SKINNY_CASE
  }
  return deep ? launch_skinny_t<8, 4, EPI>(p, st) : launch_skinny_t<4, 4, EPI>(p, st);
}

// f32 activations quantized on load (GEMM only)
template <bool CONV, int EPI>
int launch_f32a(const MainParams& p, hipStream_t st) {
  if constexpr (CONV) {
    return fail("f32 activations: GEMM only");
  } else {
    const dim3 grid((unsigned)ceil_div(p.N, 16), (unsigned)ceil_div(p.M, 16));
    DQ8_REQUIRE(grid.y <= 65535, "qgemm with f32 activations: too many rows for this kernel");
    if (p.a_round_even)
      hipLaunchKernelGGL((qgemm_skinny_f32a_kernel<8, EPI, 1>), grid, dim3(512), 0, st, p);
    else
      hipLaunchKernelGGL((qgemm_skinny_f32a_kernel<8, EPI, 0>), grid, dim3(512), 0, st, p);
    return check_hip(hipGetLastError(), "qgemm_skinny_f32a launch");
  }
}

template <bool CONV, int EPI>
int launch_variant(int variant, MainParams& p, hipStream_t st) {
  const Variant& v = kVariants[variant];
  p.tiles_m = (int)ceil_div(p.M, v.bm);
  p.tiles_n = (int)ceil_div(p.N, v.bn);
  switch (variant) {
    case 1: return launch_mfma<256, 256, 64, 2, 2, CONV, EPI>(p, st);
    case 2: return launch_mfma<128, 128, 64, 2, 2, CONV, EPI>(p, st);
    case 3: return launch_mfma<64, 64, 64, 2, 2, CONV, EPI>(p, st);
    case kPipe256: return launch_pipe<256, 256, 2, 2, 1, CONV, EPI>(p, st);
    case kPipe128: return launch_pipe<128, 128, 2, 2, 1, CONV, EPI>(p, st);
    case kPipe64: return launch_pipe<64, 64, 2, 2, 1, CONV, EPI>(p, st);
    case kPipe256x64: return launch_pipe<256, 64, 4, 1, 1, CONV, EPI>(p, st);
    case kPipe64k2: return launch_pipe<64, 64, 2, 2, 2, CONV, EPI>(p, st);
    case kPipe64k4: return launch_pipe<64, 64, 2, 2, 4, CONV, EPI>(p, st);
    case kPipe256w8: return launch_pipe<256, 256, 2, 4, 1, CONV, EPI>(p, st);
    case kPipe128w8: return launch_pipe<128, 128, 2, 4, 1, CONV, EPI>(p, st);
    case kPipe256x192: return launch_pipe<256, 192, 4, 2, 1, CONV, EPI>(p, st);
  }
  if constexpr (!CONV) {   // GEMM only: the small-M kernel and the persistent forms
    if (variant == kSkinnyVariant) return launch_skinny<EPI>(p, st);
    if (variant == kPersist256) return launch_persist<256, 256, 2, 4, false, EPI>(p, 1, st);
    if (variant == kPersist128) return launch_persist<128, 128, 2, 4, false, EPI>(p, 2, st);
    if (variant == kPersist256x192) return launch_persist<256, 192, 4, 2, false, EPI>(p, 1, st);
  }
  return fail("unknown or unsupported qgemm variant for this operation");
}

// The tiles a strided 1 x 1 convolution runs on as a GEMM over the pixels it reads (instantiated
// next to the convolution kernels: CONV true; the GEMM files carry a stub).
inline bool rowmap_has_variant(int variant) {
  return variant == kPipe128 || variant == kPipe128w8 || variant == kPipe64 || variant == kPipe64k2 ||
         variant == kPipe256w8 || variant == kPipe256x192;
}
template <bool CONV, int EPI>
int launch_rowmap(int variant, MainParams& p, hipStream_t st) {
  if constexpr (CONV) {
    const Variant& v = kVariants[variant];
    p.tiles_m = (int)ceil_div(p.M, v.bm);
    p.tiles_n = (int)ceil_div(p.N, v.bn);
    switch (variant) {
      case kPipe128: return launch_pipe<128, 128, 2, 2, 1, false, EPI, true>(p, st);
      case kPipe128w8: return launch_pipe<128, 128, 2, 4, 1, false, EPI, true>(p, st);
      case kPipe64: return launch_pipe<64, 64, 2, 2, 1, false, EPI, true>(p, st);
      case kPipe64k2: return launch_pipe<64, 64, 2, 2, 2, false, EPI, true>(p, st);
      case kPipe256w8: return launch_pipe<256, 256, 2, 4, 1, false, EPI, true>(p, st);
      case kPipe256x192: return launch_pipe<256, 192, 4, 2, 1, false, EPI, true>(p, st);
    }
  }
  return fail("no kernel with rows mapped to pixels for this variant");
}

}  // namespace dq8

// the body of one qgemm_launch_*.hip
#define DQ8_INSTANTIATE_LAUNCH(CONV, EPI) \
  namespace dq8 {                          \
  template int launch_variant<CONV, EPI>(int, MainParams&, hipStream_t); \
  template int launch_f32a<CONV, EPI>(const MainParams&, hipStream_t);   \
  template int launch_rowmap<CONV, EPI>(int, MainParams&, hipStream_t);  \
  }

#endif  // DQ8_QGEMM_LAUNCH_H_
