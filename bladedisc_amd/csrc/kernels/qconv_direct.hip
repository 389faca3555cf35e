// Host launchers of the 3x3 convolution kernels that keep the input patch in LDS.
#include "qconv_direct.h"
#include "qconv_stream.h"

#include <algorithm>

#include "dq8_common.h"
#include "disc_q8.h"

#pragma clang fp contract(off)

namespace dq8 {
namespace {

constexpr int kLdsBytes = 160 * 1024;
constexpr int kStages = 4;

struct Tile {
  int bm, bn;
};
const Tile kTiles[kNumDirectConvConfigs] = {{256, 64}, {128, 64}, {512, 64}};

template <int BM, int BN, int WM, int WN, int EPI>
int launch_t(const DirectConvParams& p, hipStream_t st) {
  const int lds = p.patch_bytes + kStages * BN * 128;
  auto kern = qconv3x3_direct_kernel<BM, BN, WM, WN, kStages, EPI>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), kLdsBytes, &lds_allowed)) return s;
  const int64_t grid = (int64_t)p.NB * p.tiles_per_image * p.tiles_n;
  DQ8_REQUIRE(grid < (1LL << 31), "direct convolution: too many tiles");
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WM * WN * 64), lds, st, p);
  return check_hip(hipGetLastError(), "qconv3x3_direct launch");
}

template <int EPI>
int launch_config(int config, const DirectConvParams& p, hipStream_t st) {
  switch (config) {
    case 0: return launch_t<256, 64, 4, 1, EPI>(p, st);
    case 1: return launch_t<128, 64, 2, 2, EPI>(p, st);
    case 2: return launch_t<512, 64, 8, 1, EPI>(p, st);
  }
  return fail("direct convolution: unknown configuration");
}

}  // namespace

void direct_conv_tile(int config, int* bm, int* bn) {
  *bm = kTiles[config].bm;
  *bn = kTiles[config].bn;
}

bool direct_conv_plan(int config, DirectConvParams* p) {
  if (config < 0 || config >= kNumDirectConvConfigs) return false;
  const int bm = kTiles[config].bm, bn = kTiles[config].bn;
  int log2_ci = 0;
  while ((1 << log2_ci) < p->Ci) ++log2_ci;
  if ((1 << log2_ci) != p->Ci || p->Ci < 16 || p->Ci > 256) return false;
  if (p->Kh < 1 || p->Kw < 1 || p->Kh > 7 || p->Kw > 7) return false;
  if (p->Ci == 16 && p->Kw % 2 != 0) return false;
  if (p->NB <= 0 || p->Ho <= 0 || p->Wo <= 0 || p->Co <= 0) return false;
  const int64_t in_bytes = (int64_t)p->NB * p->H * p->Wd * p->Ci;
  if (in_bytes >= (1LL << 31)) return false;
  // byte offset of the last weight chunk a block may address, from its first row
  if ((int64_t)(bn + 8) * p->Kh * p->Kw * p->Ci + 4 * 128 >= (1LL << 31)) return false;
  const int hw = p->Ho * p->Wo;
  const int tiles = (hw + bm - 1) / bm;
  int span = 0;
  for (int t = 0; t < tiles; ++t) {
    const int first = t * bm, last = std::min(first + bm, hw) - 1;
    span = std::max(span, last / p->Wo - first / p->Wo + 1);
  }
  const int64_t patch =
      ((int64_t)(span + p->Kh - 1) * (p->Wo + p->Kw - 1) * p->Ci + 1023) / 1024 * 1024;
  if (patch + (int64_t)kStages * bn * 128 > kLdsBytes) return false;
  // (the epilogue's staging -- 8 bytes per channel plus at most bm * bn bytes -- fits in the
  // weight stages alone: 4 * 128 * bn bytes)
  p->log2_ci = log2_ci;
  p->kw_inv = (65536 + p->Kw - 1) / p->Kw;
  p->tiles_per_image = tiles;
  p->tiles_n = (p->Co + bn - 1) / bn;
  p->patch_bytes = (int)patch;
  p->in_bytes = in_bytes;
  return true;
}

namespace {
// The (filter, slice) pairs the streaming kernel is instantiated for: 3 x 3 filters on 64 and 128
// channels, 1 x 1 filters (a GEMM over the pixels with a short k) on 64 to 256, and the 4 x 4 x 16
// form of a stem.  A slice is as wide as the registers allow -- NS K / 256 of them hold it, next
// to 16 accumulators per 32 channels of it -- since every workgroup of a pixel tile loads the
// tile's patch again; `narrow` is a second width for layers with no more output channels than
// that.  (1 x 1 x 256 with 128-channel slices spills; 1 x 1 x 512 was measured and lost to the
// GEMM tiles at every size.)
struct StreamInstance {
  int kh, kw, ci, ns, narrow;
};
constexpr StreamInstance kStreamInstances[] = {
    {3, 3, 64, 64, 0}, {3, 3, 128, 32, 0}, {1, 1, 64, 128, 64}, {1, 1, 128, 128, 0}, {4, 4, 16, 64, 0},
    {1, 1, 256, 64, 0},
};
int stream_conv_slice(int Kh, int Kw, int Ci, int Co) {
  for (const StreamInstance& s : kStreamInstances)
    if (s.kh == Kh && s.kw == Kw && s.ci == Ci) return s.narrow && Co <= s.narrow ? s.narrow : s.ns;
  return 0;
}
}  // namespace

bool stream_conv_has_instance(int Kh, int Kw, int Ci) { return stream_conv_slice(Kh, Kw, Ci, 1) != 0; }

bool stream_conv_plan(DirectConvParams* p) {
  const int ns = stream_conv_slice(p->Kh, p->Kw, p->Ci, p->Co);
  if (ns == 0) return false;
  if (p->NB <= 0 || p->Ho <= 0 || p->Wo <= 1 || p->Co <= 0) return false;
  const int K = p->Kh * p->Kw * p->Ci;
  const int64_t in_bytes = (int64_t)p->NB * p->H * p->Wd * p->Ci;
  if (in_bytes >= (1LL << 31) || (int64_t)(p->Co + ns) * K >= (1LL << 31)) return false;
  const int64_t hw = (int64_t)p->Ho * p->Wo;
  if (hw >= (1 << 24) || hw * p->Wo >= (1LL << 31)) return false;   // (exact umulhi division)
  const int64_t pitch = (p->Wo + p->Kw - 1 + 15) / 16 * 16;
  const int64_t tiles_n = ceil_div(p->Co, ns);
  const int64_t cus = compute_units();
  const int fixed = kLdsBytes - stream_conv_weight_lds(K, ns) - stream_conv_cp_bytes(ns);
  // Time of a launch in cycles of a SIMD: rounds of workgroups x (blocks of 32 pixels of the
  // busiest SIMD -- it runs waves 0 and 4, which take blocks 0, 8, ... and 4, 12, ... -- each K / 32
  // MFMAs of 32 cycles per 32 channels plus the part of their requantisation that does not
  // run under another wave's MFMAs, plus the time of loading and of the last epilogue: three
  // blocks of a 3 x 3 filter, which is the measure for the short blocks of a 1 x 1 filter too).
  const int64_t nf = ns / 32;
  const int64_t block_clk = (K / 32) * nf * 32 + nf * 230;
  const int64_t fixed_clk = p->Kh * p->Kw > 1 ? 3 * block_clk : 3 * (18 * 2 * 32 + 2 * 230);
  int64_t best_cost = -1, best_tpi = 0, best_patch = 0;
  for (int64_t tpi = 1; tpi <= ceil_div(hw, 32); ++tpi) {
    const int64_t tile = ceil_div(hw, tpi);
    if (ceil_div(hw, tile) != tpi) continue;               // the same tiling as a smaller tpi
    // image rows a tile of `tile` consecutive pixels can span, wherever it starts in a row (an
    // upper bound for this tiling, in closed form: the planner is called per launch)
    const int64_t span = std::min<int64_t>((tile + p->Wo - 2) / p->Wo + 1, p->Ho);
    // (1 x 1: the tile's pixels as they come, whole blocks of 32)
    const int64_t patch = p->Kh * p->Kw == 1
                              ? (ceil_div(tile, 32) * 32 * p->Ci + 1023) / 1024 * 1024
                              : ((span + p->Kh - 1) * pitch * p->Ci + 1023) / 1024 * 1024;
    if (patch > fixed) continue;
    const int64_t blocks = ceil_div(tile, 32);
    const int64_t simd0 = ceil_div(blocks, 8) + (blocks > 4 ? ceil_div(blocks - 4, 8) : 0);
    const int64_t wgs = (int64_t)p->NB * tpi * tiles_n;
    const int64_t cost = ceil_div(wgs, cus) * (simd0 * block_clk + fixed_clk);
    if (best_cost < 0 || cost < best_cost || (cost == best_cost && wgs <= cus)) {
      best_cost = cost;
      best_tpi = tpi;
      best_patch = patch;
    }
  }
  if (best_cost < 0) return false;
  if (((int64_t)p->NB * best_tpi + 7) / 8 * 8 * tiles_n >= (1LL << 31)) return false;
  int log2_ci = 0;
  while ((1 << log2_ci) < p->Ci) ++log2_ci;
  p->log2_ci = log2_ci;
  p->kw_inv = 0;
  p->tile_px = (int)ceil_div(hw, best_tpi);
  p->patch_pitch = (int)pitch;
  p->wo_inv = (unsigned)((1ULL << 32) / (uint64_t)p->Wo + 1);
  p->slice_n = ns;
  p->tiles_per_image = (int)best_tpi;
  p->tiles_n = (int)tiles_n;
  p->patch_bytes = (int)best_patch;
  p->in_bytes = in_bytes;
  return true;
}

namespace {
template <int KH, int KW, int CI, int NS, int EPI, bool POST>
int launch_stream_t(const DirectConvParams& p, hipStream_t st) {
  const int lds = p.patch_bytes + stream_conv_weight_lds(KH * KW * CI, NS) + stream_conv_cp_bytes(NS);
  auto kern = qconv_stream_kernel<KH, KW, CI, NS, EPI, POST>;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int s = allow_dynamic_lds(reinterpret_cast<const void*>(kern), kLdsBytes, &lds_allowed)) return s;
  // (pixel tiles rounded up to a multiple of 8: workgroup b works on tile 8 (b / 8 / slices) + b % 8)
  const int64_t tiles = ((int64_t)p.NB * p.tiles_per_image + 7) / 8 * 8;
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles * p.tiles_n)), dim3(512), lds, st, p);
  return check_hip(hipGetLastError(), "qconv_stream launch");
}

template <int KH, int KW, int CI, int NS, int EPI>
int launch_stream_post(const DirectConvParams& p, hipStream_t st) {
  const bool post = p.epi.table != nullptr || p.epi.resid_kind != 0;
  return post ? launch_stream_t<KH, KW, CI, NS, EPI, true>(p, st)
              : launch_stream_t<KH, KW, CI, NS, EPI, false>(p, st);
}

template <int EPI>
int launch_stream_epi(const DirectConvParams& p, hipStream_t st) {
  const int taps = p.Kh * p.Kw;
  if (taps == 9 && p.Ci == 64 && p.slice_n == 64) return launch_stream_post<3, 3, 64, 64, EPI>(p, st);
  if (taps == 9 && p.Ci == 128 && p.slice_n == 32) return launch_stream_post<3, 3, 128, 32, EPI>(p, st);
  if (p.Kh == 4 && p.Kw == 4 && p.Ci == 16 && p.slice_n == 64) return launch_stream_post<4, 4, 16, 64, EPI>(p, st);
  if (taps == 1 && p.Ci == 64 && p.slice_n == 128) return launch_stream_post<1, 1, 64, 128, EPI>(p, st);
  if (taps == 1 && p.Ci == 64 && p.slice_n == 64) return launch_stream_post<1, 1, 64, 64, EPI>(p, st);
  if (taps == 1 && p.Ci == 128 && p.slice_n == 128) return launch_stream_post<1, 1, 128, 128, EPI>(p, st);
  // (256 channels: without fused operators only -- with them the kernel would spill)
  if (taps == 1 && p.Ci == 256 && !(p.epi.table != nullptr || p.epi.resid_kind != 0)) {
    if (p.slice_n == 64) return launch_stream_t<1, 1, 256, 64, EPI, false>(p, st);
  }
  return fail("the streaming convolution kernel has no instance for this filter");
}
}  // namespace

int launch_stream_conv(int epilogue, const DirectConvParams& p, hipStream_t st) {
  switch (epilogue) {
    case DQ8_EPI_REQUANT_CPU: return launch_stream_epi<DQ8_EPI_REQUANT_CPU>(p, st);
    case DQ8_EPI_REQUANT_GPU: return launch_stream_epi<DQ8_EPI_REQUANT_GPU>(p, st);
  }
  return fail("the streaming convolution kernel has int8 results only");
}

int launch_direct_conv(int config, int epilogue, const DirectConvParams& p, hipStream_t st) {
  switch (epilogue) {
    case DQ8_EPI_ACC_S32: return launch_config<DQ8_EPI_ACC_S32>(config, p, st);
    case DQ8_EPI_REQUANT_CPU: return launch_config<DQ8_EPI_REQUANT_CPU>(config, p, st);
    case DQ8_EPI_REQUANT_GPU: return launch_config<DQ8_EPI_REQUANT_GPU>(config, p, st);
    case DQ8_EPI_DEQUANT_F32: return launch_config<DQ8_EPI_DEQUANT_F32>(config, p, st);
  }
  return fail("unknown epilogue");
}

}  // namespace dq8
