// int8 NHWC stride-1 convolution (3x3 in the first place) with the input patch resident in LDS.
//
// As an implicit GEMM a 3x3 convolution pulls every input pixel through the CU's
// address unit nine times (once per tap), and at 64 or 128 channels that, not the MFMAs,
// sets the pace (144 KiB of operand loads per 256 output pixels at Ci = 64 against 2300
// MFMA cycles).  Here a workgroup computes 256 consecutive output pixels of one image
// (row-major, so they span a few full image rows) for BN output channels:
//  * the input rows those pixels touch, with a one-pixel frame (zeros where the frame is
//    padding), are loaded into LDS once -- 30 KiB instead of 144 KiB for a 56-wide image
//    with 64 channels -- by direct-to-LDS loads;
//  * the activation fragment of tap (kh, kw) is read from that patch at the pixel's
//    position shifted by (kh, kw); 16-byte channel chunk c of patch pixel q sits in slot
//    c ^ f(q), f chosen so that 16 consecutive pixels reading the same chunk cover all
//    64 banks (conflict-free ds_read_b128);
//  * the weights [Co, 3, 3, Ci] stream through NS LDS stages in k tiles of 128, laid out
//    as in the GEMM kernel (8-row x 128-byte blocks, the same swizzle), k running over
//    (kh, kw, ci); chunks past K load zeros.  NS - 1 tiles are in flight: the weights come
//    from the L2, and one tile of MFMAs (a few hundred cycles) does not cover that trip.
//    (Loading a workgroup's whole weight slice up front instead -- 36 KiB for 64 channels
//    in and out, a k loop without waits or barriers -- was measured: the k loop gets 12 %
//    shorter, the launch no faster.  Eight waves instead of four on the 256 x 64 tile:
//    slower at 64 channels, 9.75 against 10.7 us at 128, where the implicit GEMM is used.)
// Requires Ci in {32, 64, 128, 256}, 16-byte aligned tensors, dilation 1, stride 1.  Other
// filter sizes up to 7 x 7 run the same way (k runs over (kh, kw, ci), the patch has Kh - 1
// and Kw - 1 extra rows and columns), and so do 16 channels with an even filter width: the 32
// bytes of k of an MFMA step are then two taps next to each other in a filter row, i.e. two
// neighbouring patch pixels -- the stride-1 form of a stem convolution after space to depth.
#ifndef DQ8_QCONV_DIRECT_H_
#define DQ8_QCONV_DIRECT_H_

#include "qgemm_pipelined.h"

namespace dq8 {

struct DirectConvParams {
  const int8_t* in;     // [NB, H, W, Ci]
  const int8_t* w;      // [Co, Kh, Kw, Ci]
  int NB, H, Wd, Ci, Co, Ho, Wo;
  int Kh, Kw;
  int kw_inv;           // ceil(65536 / Kw): tap / Kw == (tap * kw_inv) >> 16 for tap < 64
  int pad_t, pad_l;
  int log2_ci;          // Ci = 1 << log2_ci
  int tile_px;          // output pixels per tile where that is not a template parameter
  int patch_pitch;      // (streaming kernel) pixels per patch row in LDS: Wo + Kw - 1 rounded up to 16
  unsigned wo_inv;      // (streaming kernel) floor(2^32 / Wo) + 1: pixel / Wo == umulhi(pixel, wo_inv)
  int slice_n;          // (streaming kernel) output channels per workgroup
  int tiles_per_image;  // ceil(Ho * Wo / BM)
  int tiles_n;          // ceil(Co / BN)
  int patch_bytes;      // LDS reserved for the patch: (most rows a tile spans + Kh - 1) *
                        // (Wo + Kw - 1) * Ci, rounded up to 1 KiB
  int64_t in_bytes;
  EpiParams epi;
};

template <int BM, int BN, int WM, int WN, int NS, int EPI>
__global__ void __launch_bounds__(WM* WN * 64) qconv3x3_direct_kernel(const DirectConvParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BK = 128;
  constexpr int NW = WM * WN;
  constexpr int NT = NW * 64;
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int FM = TM / 32, FN = TN / 32;
  constexpr int B_BYTES = BN * BK;
  constexpr int B_LD = (BN / 8) / NW;
  constexpr int kOutOfRange = (int)0x80000000;
  static_assert(NW % 2 == 0 && (BN / 8) % NW == 0, "the weight tile splits over the waves");
  static_assert(FM >= 1 && FN >= 1, "fragment mismatch");
  static_assert(NS >= 2 && B_LD * (NS - 1) <= 63, "vmcnt is a 6-bit counter");

  extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
  DQ8_TRACE_POINT(0);
  int8_t* patch = smem;                       // [patch pixels][Ci], chunks swizzled;
                                              // the weight stages follow it

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  // block -> (image, pixel tile, channel tile); channel tiles of one pixel tile are
  // neighbours so that they find the same input rows in the L2
  const int tn = blockIdx.x % p.tiles_n;
  const int rest = blockIdx.x / p.tiles_n;
  const int tp = rest % p.tiles_per_image;
  const int img = rest / p.tiles_per_image;
  const int n0 = tn * BN;
  const int hw = p.Ho * p.Wo;
  const int p0 = tp * BM;                                  // first output pixel of the tile
  const int p_last = min(p0 + BM, hw) - 1;
  const int y_base = p0 / p.Wo;
  const int rows = p_last / p.Wo - y_base + p.Kh;          // patch rows in use
  const int PW = p.Wo + p.Kw - 1;                          // patch width
  const int taps = p.Kh * p.Kw;
  const int CP = p.Ci >> 4;                                // 16-byte chunks per pixel
  // LDS swizzle: chunk c of patch pixel q is stored in slot c ^ f(q) of the pixel.  A
  // 16-byte-per-lane LDS read is served 16 lanes (256 bytes, all 64 banks) at a time; the
  // 16 lanes read the same chunk of 16 consecutive pixels, and f makes those 16 slots fall
  // into 16 different 16-byte columns of the 256-byte bank row (measured on one wave: 27.0
  // cycles per read like a linear pattern, 38 without the swizzle):
  // f(q) = (q >> fshift) & fmask.
  const int fshift = p.log2_ci >= 8 ? 0 : 8 - p.log2_ci;
  const int fmask = CP - 1;
  const int KT = (taps * p.Ci + BK - 1) / BK;

  const v4i in_rsrc = make_rsrc(p.in, p.in_bytes);
  const int8_t* w_base = p.w + (int64_t)n0 * taps * p.Ci;
  const int64_t w_valid = (int64_t)(p.Co - n0) * taps * p.Ci;
  const v4i w_rsrc = make_rsrc(w_base, w_valid < 0x7fffffff ? w_valid : 0x7fffffff);
  const unsigned lds_base =
      (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(size_t)(lds_void_t*)smem);

  // ---- the patch: instruction j of the workgroup fills LDS bytes [1024 j, 1024 j + 1024),
  // lane l the 16-byte chunk g = 64 j + l.  A wave's instructions are NW apart, so its
  // lane's patch pixel advances by the same step every time: (row, column) are carried
  // along instead of divided out again.
  {
    const int lcp = p.log2_ci - 4;
    const int total = rows * PW * CP;                      // chunks in use
    const int img_px = img * p.H * p.Wd;
    const int dq = (NW * 64) >> lcp;                       // pixels per step
    const int dq_y = dq / PW, dq_x = dq - dq_y * PW;
    int g = wave * 64 + lane;
    int q = g >> lcp;
    int hy = q / PW, hx = q - hy * PW;
    const int slot = g & (CP - 1);                         // NW * 64 is a multiple of CP
    for (int j = wave; j * 64 < total; j += NW) {
      const int c = slot ^ ((q >> fshift) & fmask);        // channel chunk stored in this slot
      const int iy = y_base - p.pad_t + hy, ix = hx - p.pad_l;
      const bool ok = g < total && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.Wd;
      const int voff = ok ? ((img_px + iy * p.Wd + ix) << p.log2_ci) + (c << 4) : kOutOfRange;
      buffer_load_lds_b128(in_rsrc, (unsigned)__builtin_amdgcn_readfirstlane((int)(lds_base + j * 1024)),
                           voff);
      g += NW * 64;
      q += dq;
      hx += dq_x;
      hy += dq_y;
      if (hx >= PW) {
        hx -= PW;
        ++hy;
      }
    }
  }

  // ---- weight tile loads: as in the GEMM kernel
  const int lr = lane >> 3, ls = lane & 7;
  const int kc = (ls ^ lr ^ (wave & 1)) << 4;
  int b_off[B_LD], b_lds[B_LD];
#pragma unroll
  for (int i = 0; i < B_LD; ++i) {
    const int qb = wave + i * NW;
    b_off[i] = (qb * 8 + lr) * taps * p.Ci + kc;
    b_lds[i] = __builtin_amdgcn_readfirstlane(p.patch_bytes + qb * 1024);
  }
  auto issue_weights = [&](int kt, int st) {
    const bool in = kt < KT && kt * BK + kc < taps * p.Ci;
    const unsigned base = (unsigned)__builtin_amdgcn_readfirstlane((int)(lds_base + st * B_BYTES));
#pragma unroll
    for (int i = 0; i < B_LD; ++i)
      buffer_load_lds_b128(w_rsrc, base + b_lds[i], in ? b_off[i] + kt * BK : kOutOfRange);
  };

  // ---- per-fragment pixel positions in the patch (tap (0, 0))
  int hq[FM];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    int px = p0 + wm * TM + i * 32 + (lane & 31);
    px = px < hw ? px : hw - 1;                            // rows past the image are not stored
    const int y = px / p.Wo, x = px - y * p.Wo;
    hq[i] = (y - y_base) * PW + x;
  }
  const int row_in_frag = lane & 31;
  const int swz = (lane & 7) ^ ((lane >> 3) & 1);
  const int b_frag0 = p.patch_bytes + (wn * TN / 8) * 1024 + (row_in_frag >> 3) * 1024 + (lane & 7) * 128;

  v16i acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

#pragma unroll
  for (int t = 0; t < NS - 1; ++t) issue_weights(t, t);
  // The per-channel epilogue factors are fetched behind the patch and the first weight
  // tiles, so that their cold loads travel together with those instead of ahead of them.
  EarlyColParams<EPI, NT, BN> early;
  early.fetch(p.epi, n0);

  // Fragments are read one k-step ahead of their MFMAs, into two alternating sets.
  v4i fa[2][FM], fb[2][FN];
  auto load_frags = [&](int set, int kt, int st, int ks) {
    // the 32 bytes of k of a step lie in one tap (Ci a multiple of 32) or in two taps next to
    // each other in a filter row (Ci = 16, even Kw: chunk 1 of a 16-byte pixel is the next one)
    const int koff = kt * BK + ks * 32;
    int tap = koff >> p.log2_ci;
    tap = tap < taps ? tap : taps - 1;                     // past K: the weights are zeros
    const int kh = (tap * p.kw_inv) >> 16, kw = tap - p.Kw * kh;
    const int c = ((koff & (p.Ci - 1)) >> 4) + (lane >> 5);
    const int shift = kh * PW + kw;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int q = hq[i] + shift;
      fa[set][i] = *(const v4i*)(patch + (q << p.log2_ci) + ((c ^ ((q >> fshift) & fmask)) << 4));
    }
#pragma unroll
    for (int j = 0; j < FN; ++j)
      fb[set][j] = *(const v4i*)(smem + st * B_BYTES + b_frag0 + j * 4096 +
                                 (((2 * ks + (lane >> 5)) ^ swz) << 4));
  };

  // The patch and tile 0 have landed once all loads but those of the NS - 2 newest tiles
  // are done -- for this wave; after the barrier for all.
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(B_LD * (NS - 2)));
  __syncthreads();
  DQ8_TRACE_POINT(1);
  issue_weights(NS - 1, NS - 1);
  load_frags(0, 0, 0, 0);

  int cur = 0;
  for (int kt = 0; kt < KT; ++kt) {
    const int nxt = cur == NS - 1 ? 0 : cur + 1;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      if (ks < 3) {
        load_frags((ks + 1) & 1, kt, cur, ks + 1);
      } else {
        // This wave has read all it needs of tile kt, and tile kt + 1 (all loads but those
        // of the NS - 2 newest tiles) has landed for it; after the barrier that holds for
        // every wave: stage `cur` takes tile kt + NS, stage `nxt` can be read.  (Tiles past
        // the last are issued too -- as zeros, touching no memory -- so that the count of
        // loads in flight stays the same.)
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(B_LD * (NS - 2)));
        __syncthreads();
        issue_weights(kt + NS, cur);
        load_frags(0, kt + 1, nxt, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks & 1][j], fa[ks & 1][i], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    cur = nxt;
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  DQ8_TRACE_POINT(2);

  const int m_img0 = img * hw;
  mfma_epilogue<EPI, FM, FN, NT, BN>(acc, p.epi, smem, m_img0 + p0 + wm * TM, n0 + wn * TN, n0,
                                     early.c, -1, true, m_img0 + hw);
  DQ8_TRACE_POINT(3);
#else
  (void)p;
#endif
}

// ---- host side (qconv_direct.hip)
constexpr int kNumDirectConvConfigs = 3;

// Tile shape of configuration `config` (0 .. kNumDirectConvConfigs - 1).
void direct_conv_tile(int config, int* bm, int* bn);

// Whether configuration `config` can run the problem: filter up to 7 x 7 (p->Kh, p->Kw), Ci in
// {32, 64, 128, 256} or 16 with an even Kw, 32-bit buffer offsets, and the patch plus the weight
// stages fit the LDS.  Fills the
// launch geometry of `p` (tiles_per_image, tiles_n, patch_bytes, log2_ci).
bool direct_conv_plan(int config, DirectConvParams* p);

// Launches configuration `config` on a planned problem; 0 or an error status.
int launch_direct_conv(int config, int epilogue, const DirectConvParams& p, hipStream_t st);

}  // namespace dq8

#endif  // DQ8_QCONV_DIRECT_H_
