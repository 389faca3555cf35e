// Host launchers of the 3x3 convolution kernels that keep the input patch in LDS.
#include "qconv_direct.h"

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
