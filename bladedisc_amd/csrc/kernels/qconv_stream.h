// int8 NHWC stride-1 convolution with the whole filter in registers ("streaming" form), for
// filters of which a slice of NS output channels fits there: NS * Kh * Kw * Ci <= 36 KiB
// (3 x 3 x 64 with 64-channel slices in the first place, 3 x 3 x 128 with 32-channel slices,
// 1 x 1 x 64 and 1 x 1 x 128 with 128-channel slices, 1 x 1 x 256 with 64-channel slices,
// 4 x 4 x 16 -- a 7 x 7 stride-2 stem after
// space to depth -- with 64-channel slices).
//
// Where the time of such a layer goes in the LDS-tiled kernels (32 x 56 x 56 x 64 -> 64, 9 us):
// every workgroup loads, then multiplies, then requantises and stores, all in the same phase, so
// the matrix pipe idles while operands arrive and while the epilogue's VALU chain runs (a wave
// issues about one VALU instruction per 5 cycles; 64 results per lane are 1.3 us of it), and the
// k loop itself is paced by barriers and by LDS reads of both operands.  Here
//  * a workgroup (8 waves, one per compute unit) takes `tile_px` consecutive output pixels of one
//    image x NS output channels (the slices of one pixel tile run on the same XCD, so that its
//    L2 fetches their common patch once); the input rows they touch, with the filter's frame, are loaded
//    into LDS once (as in qconv_direct.h, same swizzle);
//  * the NS x K weight slice is loaded into LDS once and from there into registers: every wave
//    holds all of it in MFMA operand layout (NS K / 256 registers: 144 for 3 x 3 x 64), so the
//    main loop reads only the pixel operand from LDS -- 1 KiB per NS / 32 MFMAs -- and has no
//    barrier;
//  * a wave walks blocks of 32 pixels: K / 32 steps of NS / 32 MFMAs (one per 32 channels), then
//    requantises and stores that block's 32 x NS results from registers and goes on to its next
//    block.  The two waves of a SIMD drift apart by themselves (the older wave wins the matrix
//    pipe), so one wave's epilogue runs under the other's MFMAs.
// The weights go to LDS before the patch and are copied to registers while the patch is still
// arriving.
// A 1 x 1 filter (a GEMM over the pixels with k = Ci) runs the same way on 64 to 256 channels,
// where the GEMM kernels' k tile of 128 is short or half empty and their lock-step
// requantisation is most of the time; its blocks share no pixels, so a wave loads those of its
// own blocks and waits for no other wave's: the first block's before the weights' barrier, the
// others' while the first is multiplied.
// int8 results only (REQUANT_CPU / REQUANT_GPU, with or without the fused operators of
// dq8_qconv2d_fused), 16-byte aligned output rows.
#ifndef DQ8_QCONV_STREAM_H_
#define DQ8_QCONV_STREAM_H_

#include "qconv_direct.h"

// Per-wave timeline hook for profiling builds, like DQ8_TRACE_POINT: stage i of the calling wave
// (0 entry, 1 weights in LDS, 2 weights in registers, 3 patch landed, 4 + 2 k / 5 + 2 k: MFMAs /
// stores of the wave's k-th block done).  Expands to nothing in the library.
#ifndef DQ8_TRACE_WAVE
#define DQ8_TRACE_WAVE(i)
#endif

namespace dq8 {

// LDS bytes the kernel needs on top of the patch: the padded weight slice (rows of K + 16
// bytes, rounded up to the 8 KiB the eight waves' equal shares of load instructions cover) and
// the per-channel (scale, addend) pairs.
constexpr int stream_conv_weight_lds(int K, int NS) {
  return ((NS * (K / 16 + 1) + 511) / 512) * 512 * 16;
}
// (the per-channel factors, a fused table, and -- from 64 channels a slice on -- a 32 x NS result
// tile per wave)
constexpr int stream_conv_cp_bytes(int NS) { return NS * 8 + 256 + (NS >= 64 ? 8 * 32 * NS : 0); }

// POST: the launch has operators fused behind the convolution (their code and registers are kept
// out of the plain form).
template <int KH, int KW, int CI, int NS, int EPI, bool POST>
__global__ void __launch_bounds__(512) qconv_stream_kernel(const DirectConvParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  static_assert(EPI == DQ8_EPI_REQUANT_CPU || EPI == DQ8_EPI_REQUANT_GPU, "int8 results only");
  static_assert(CI == 16 || CI == 32 || CI == 64 || CI == 128 || CI == 256 || CI == 512, "channels per pixel");
  static_assert(CI >= 32 || KW % 2 == 0, "16 channels: an MFMA step takes two taps next to each other");
  constexpr int NW = 8;
  constexpr int K = KH * KW * CI;
  constexpr int KS = K / 32;                 // MFMA steps per block
  constexpr int ROWC = K / 16 + 1;           // 16-byte chunks per weight row in LDS (one of padding)
  constexpr int NF = NS / 32;                // 32-channel fragments of the slice
  constexpr int W_INSTR = (NS * ROWC + 63) / 64;           // 1 KiB load instructions for the slice
  constexpr int W_PER_WAVE = (W_INSTR + NW - 1) / NW;      // every wave issues this many
  constexpr int W_LDS = stream_conv_weight_lds(K, NS);
  constexpr int LOG2_CI = CI == 16 ? 4 : CI == 32 ? 5 : CI == 64 ? 6 : CI == 128 ? 7 : CI == 256 ? 8 : 9;
  constexpr int CP = CI / 16;                // 16-byte chunks per pixel
  // (swizzle of the chunks inside a 256-byte bank row, as in qconv_direct.h)
  constexpr int FSHIFT = LOG2_CI >= 8 ? 0 : 8 - LOG2_CI, FMASK = CP > 16 ? 15 : CP - 1;
  constexpr int STEPS_PER_TAP = CI >= 32 ? CI / 32 : 1;
  constexpr int kOutOfRange = (int)0x80000000;
  // Results leave through a wave-private LDS tile where a slice row is 64 bytes or more: of a
  // fragment a lane pair holds 32 bytes of a pixel's row; read back in row order, a store
  // instruction covers whole 64- or 128-byte pieces, which can be written through the L2 (see
  // st_through: an ordinary store's dirty lines are written back after the kernel's last wave,
  // 25 MB of results in about 2.5 us; 32-byte pieces written through are slower than that).
  // Not where the fused operators come on top of a filter slice of 144 registers: no room.
  constexpr bool STAGE = NS >= 64 && !(POST && KS * NF * 4 + NF * 16 > 170);
  constexpr int LPR = NS / 16;                // lanes (16-byte chunks) per row of that tile
  // The factors of a lane's channels (16 scales and 16 addends per 32-channel fragment) stay in
  // registers over all blocks where the filter slice leaves room for them; otherwise they are
  // read from LDS per fragment, all reads of a fragment ahead of its arithmetic (read one by one
  // as they are needed, each read exposes the LDS latency under the other waves' fragment reads).
  constexpr bool HOIST_OS = KS * NF * 4 + NF * 16 + NF * 16 + 60 <= 240;
  constexpr bool HOIST_B = KS * NF * 4 + NF * 16 + NF * 32 + 60 <= 240;
  static_assert(W_PER_WAVE * NW * 1024 <= W_LDS, "weight area");
  static_assert(NS % 32 == 0 && K % 32 == 0 && KS * NF * 4 <= 160, "the filter slice must fit the registers");

  extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
  DQ8_TRACE_POINT(0);
  DQ8_TRACE_WAVE(0);
  int8_t* patch = smem;
  int8_t* wlds = smem + p.patch_bytes;
  // per-channel factors: the scales, then the addends (a launch without bias and zero point
  // reads only the first)
  float* cp_os = reinterpret_cast<float*>(smem + p.patch_bytes + W_LDS);
  float* cp_b = cp_os + NS;
  uint8_t* tab = reinterpret_cast<uint8_t*>(smem + p.patch_bytes + W_LDS + NS * 8);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const EpiParams& e = p.epi;

  // workgroup -> (pixel tile, channel slice): consecutive workgroups go to the 8 XCDs in turn,
  // so workgroups 8 apart share an L2; those are given the slices of one pixel tile
  const int xcd = blockIdx.x & 7, r8 = blockIdx.x >> 3;
  const int tn = r8 % p.tiles_n;
  const int rest = (r8 / p.tiles_n) * 8 + xcd;
  if (rest >= p.NB * p.tiles_per_image) return;            // (the grid is rounded up to 8 tiles)
  const int tp = rest % p.tiles_per_image;
  const int img = rest / p.tiles_per_image;
  const int n0 = tn * NS;
  const int hw = p.Ho * p.Wo;
  const int p0 = tp * p.tile_px;                           // first output pixel of the tile
  const int p_end = min(p0 + p.tile_px, hw);
  const int y_base = p0 / p.Wo;
  const int rows = (p_end - 1) / p.Wo - y_base + KH;       // patch rows in use
  const int PW = p.Wo + KW - 1;

  const v4i in_rsrc = make_rsrc(p.in, p.in_bytes);
  const int8_t* w_base = p.w + (int64_t)n0 * K;
  const int64_t w_valid = (int64_t)(p.Co - n0) * K;
  const v4i w_rsrc = make_rsrc(w_base, w_valid < 0x7fffffff ? w_valid : 0x7fffffff);
  const unsigned lds_base =
      (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(size_t)(lds_void_t*)smem);

  // ---- per-channel factors: the loads go out first and are used last
  ColRaw raw = {1.0f, 1.0f, 1.0f, 0};
  if (tid < NS) raw = col_fetch<EPI>(e, n0 + tid < e.N ? n0 + tid : e.N - 1);
  uint32_t tab_word = 0;
  if (POST && e.table && tid >= 64 && tid < 128)      // (a fused table: 256 bytes, fetched by wave 1)
    tab_word = reinterpret_cast<const uint32_t*>(e.table)[tid - 64];

  // ---- the weight slice: LDS rows of ROWC chunks, chunk g = 64 j + lane of instruction j
#pragma unroll
  for (int i = 0; i < W_PER_WAVE; ++i) {
    const int j = wave + i * NW;
    const int g = j * 64 + lane;
    const int row = g / ROWC, c = g - row * ROWC;
    const bool ok = row < NS && c < K / 16;
    buffer_load_lds_b128(w_rsrc, lds_base + p.patch_bytes + j * 1024,
                         ok ? row * K + (c << 4) : kOutOfRange);
  }

  // ---- the patch.  1 x 1 filter: a wave loads the pixels of its own blocks, block by block, and
  // waits for no other wave's (pixel t of the tile at LDS bytes [CI t, CI t + CI), chunks swizzled)
  constexpr bool POINT = KH == 1 && KW == 1;
  constexpr int IPB = CI / 32;                             // load instructions per block of 32 pixels
  const int nblocks = (p_end - p0 + 31) >> 5;
  const int PWp = p.patch_pitch;
  int n_patch;                       // patch load instructions of this wave issued ahead of the weights' wait
  auto load_block = [&](int b) {
#pragma unroll
    for (int i = 0; i < IPB; ++i) {
      const int g = i * 64 + lane;
      const int t = b * 32 + (g >> (LOG2_CI - 4));
      const int c = (g & (CP - 1)) ^ ((t >> FSHIFT) & FMASK);
      const int voff = p0 + t < p_end ? ((img * hw + p0 + t) << LOG2_CI) + (c << 4) : kOutOfRange;
      buffer_load_lds_b128(in_rsrc,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(lds_base + (b * 32 << LOG2_CI) + i * 1024)),
                           voff);
    }
  };
  if constexpr (POINT) {
    // (the first block now; the others once the per-channel factors, whose loads the compiler
    // waits for with a count that knows nothing of these, have been used)
    n_patch = 0;
    if (wave < nblocks) {
      load_block(wave);
      n_patch = IPB;
    }
  } else {
    // instruction j of the workgroup fills LDS bytes [1024 j, 1024 j + 1024); patch
    // rows have a pitch of PWp pixels, a multiple of 16, so that a step down a row leaves the
    // swizzle of a pixel as it is (the pixels between the frame and the pitch are never read)
    const int total = rows * PWp * CP;                       // chunks in use
    n_patch = (((total + 63) >> 6) - wave + NW - 1) / NW;
    const int img_px = img * p.H * p.Wd;
    constexpr int dq = (NW * 64) >> (LOG2_CI - 4);         // pixels per step
    const int dq_y = dq / PWp, dq_x = dq - dq_y * PWp;
    int g = wave * 64 + lane;
    int q = g >> (LOG2_CI - 4);
    int hy = q / PWp, hx = q - hy * PWp;
    const int slot = g & (CP - 1);
    for (int j = wave; j * 64 < total; j += NW) {
      const int c = slot ^ ((q >> FSHIFT) & FMASK);
      const int iy = y_base - p.pad_t + hy, ix = hx - p.pad_l;
      const bool ok = g < total && hx < PW && (unsigned)iy < (unsigned)p.H &&
                      (unsigned)ix < (unsigned)p.Wd;
      const int voff = ok ? ((img_px + iy * p.Wd + ix) << LOG2_CI) + (c << 4) : kOutOfRange;
      buffer_load_lds_b128(in_rsrc, (unsigned)__builtin_amdgcn_readfirstlane((int)(lds_base + j * 1024)),
                           voff);
      g += NW * 64;
      q += dq;
      hx += dq_x;
      hy += dq_y;
      if (hx >= PWp) {
        hx -= PWp;
        ++hy;
      }
    }
  }

  // ---- this wave's weight loads are the oldest in flight: they have landed once at most its
  // patch loads remain.  (Weights from one half of the waves and the patch from the other, so
  // that neither queues behind the other, was measured: both land 0.5 us later.)
  auto wait_patch_loads = [&](int left) {   // until at most `left` of this wave's loads are in flight
    constexpr int kMost = POINT ? 32 : 12;
    if (left >= kMost) {
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kMost));
    } else {
      static_for<kMost>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        if (left == k) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(k));
      });
    }
  };
  wait_patch_loads(n_patch);
  __syncthreads();          // the weights are in LDS
  DQ8_TRACE_WAVE(1);

  // ---- weights into registers, MFMA operand layout: lane l holds channel l % 32 of a
  // 32-channel group and the 16 bytes of k at 32 s + 16 (l / 32)
  v4i wreg[KS][NF];
  {
    const int8_t* wl = wlds + ((lane & 31) * ROWC + (lane >> 5)) * 16;
    static_for<KS>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      static_for<NF>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        wreg[s][j] = *reinterpret_cast<const v4i*>(wl + j * 32 * ROWC * 16 + s * 32);
      });
    });
  }

  DQ8_TRACE_WAVE(2);
  // ---- everything has landed for this wave (1 x 1: all but its own pixels, which no other
  // wave reads); the factors are worked out and parked
  if constexpr (!POINT) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  if (tid < NS) {
    const ColParams c = col_finish<EPI>(e, raw);
    cp_os[tid] = c.os;
    cp_b[tid] = c.b;
  }
  if (POST && e.table && tid >= 64 && tid < 128) reinterpret_cast<uint32_t*>(tab)[tid - 64] = tab_word;
  int later = 0;                     // (1 x 1) load instructions of this wave's blocks after the current one
  if constexpr (POINT) {
    for (int b = wave + NW; b < nblocks; b += NW) {
      load_block(b);
      later += IPB;
    }
  }
  __syncthreads();
  DQ8_TRACE_POINT(1);
  DQ8_TRACE_WAVE(3);

  const bool plain = e.bias_kind == DQ8_BIAS_NONE && e.zo == 0;
  int8_t* out = static_cast<int8_t*>(e.out);
  const int c0 = lane >> 5;
  const int pitch_bytes = PWp << LOG2_CI;
  int8_t* stg = reinterpret_cast<int8_t*>(tab) + 256 + wave * (32 * NS);
  // lane's channels of fragment j: j * 32 + 4 * c0 + 8 * g + 0 .. 3, g = 0 .. 3
  v4f hos[HOIST_OS ? NF : 1][4], hb[HOIST_B ? NF : 1][4];
  if constexpr (HOIST_OS) {
    static_for<NF>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
#pragma unroll
      for (int g = 0; g < 4; ++g) hos[j][g] = *reinterpret_cast<const v4f*>(&cp_os[j * 32 + 4 * c0 + 8 * g]);
    });
  }
  if constexpr (HOIST_B) {
    if (!plain) {
      static_for<NF>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
#pragma unroll
        for (int g = 0; g < 4; ++g) hb[j][g] = *reinterpret_cast<const v4f*>(&cp_b[j * 32 + 4 * c0 + 8 * g]);
      });
    }
  }

  for (int b = wave; b < nblocks; b += NW) {
    // this lane's pixel: position in the patch at tap (0, 0)
    const int px_raw = p0 + b * 32 + (lane & 31);
    int hq;
    if constexpr (POINT) {
      hq = b * 32 + (lane & 31);
      wait_patch_loads(later);        // the block's pixels have landed (later blocks' may be on their way)
      later -= IPB;
    } else {
      const int px = px_raw < p_end ? px_raw : p_end - 1;
      const int y = (int)__umulhi((unsigned)px, p.wo_inv), x = px - y * p.Wo;
      hq = (y - y_base) * PWp + x;
    }
    // byte offset of this lane's 16 bytes of k-half 0 at filter column kw, filter row 0; k-half
    // h is the same with bit 5 + ... flipped (xor 32 h), filter row kh adds kh row pitches
    int a0[KW];
    if constexpr (CI == 16) {
      a0[0] = (hq + c0) << 4;
    } else {
#pragma unroll
      for (int kw = 0; kw < KW; ++kw) {
        const int q = hq + kw;
        a0[kw] = (q << LOG2_CI) + ((c0 ^ ((q >> FSHIFT) & FMASK)) << 4);
      }
    }

    // pixel fragments, read PF steps ahead of their MFMAs
    constexpr int PF = NF >= 2 ? 4 : 7;
    v4i fa[8];
    auto load_frag = [&](auto sc) {
      constexpr int s = decltype(sc)::value;
      if constexpr (CI == 16) {
        // a pixel is one chunk (no swizzle): the step's 32 bytes of k are the taps 2 j and
        // 2 j + 1 of a filter row, i.e. two neighbouring patch pixels, one per half-wave
        constexpr int kh = s / (KW / 2), j = s - (KW / 2) * kh;
        fa[s & 7] = *reinterpret_cast<const v4i*>(patch + a0[0] + 32 * j + kh * pitch_bytes);
      } else {
        constexpr int tap = s / STEPS_PER_TAP;
        constexpr int kh = tap / KW, kw = tap - KW * kh;
        constexpr int h = s % STEPS_PER_TAP;
        fa[s & 7] = *reinterpret_cast<const v4i*>(patch + (a0[kw] ^ (32 * h)) + kh * pitch_bytes);
      }
    };
    static_for<PF>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      if constexpr (s < KS) load_frag(IntC<s>());
    });
    // (A 32-channel slice is one chain of MFMAs, each waiting for the one before it -- 48.6
    // cycles apiece instead of 32 for a wave on its own; even and odd steps on two accumulators
    // were measured on one box: 32 x 28 x 28 x 128 -> 128 8.63 against 8.74 us -- the other wave
    // of the SIMD fills the gaps already; not worth 16 more registers.)
    v16i acc[NF];
    static_for<KS>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      if constexpr (s + PF < KS) load_frag(IntC<s + PF>());
      __builtin_amdgcn_sched_barrier(0);
      static_for<NF>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        if constexpr (s == 0) {
          // (the accumulators start from the instruction's constant zero, not from moves)
          const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[s][j], fa[s & 7], zero, 0, 0, 0);
        } else {
          acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[s][j], fa[s & 7], acc[j], 0, 0, 0);
        }
      });
      __builtin_amdgcn_sched_barrier(0);
    });

    DQ8_TRACE_WAVE(4 + 2 * ((b - wave) / NW));
    // ---- requantise and store the block's 32 x NS results: of a 32 x 32 fragment a lane holds
    // pixel lane % 32 and the channel quads 8 g + 4 (lane / 32) .. + 3; two half-wave swaps
    // leave it with 16 consecutive channels, one 16-byte store
    const int64_t m = (int64_t)img * hw + px_raw;
    auto finish = [&](auto mode_c) {
      constexpr bool PLAIN = decltype(mode_c)::value == 1;
      static_for<NF>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const int cl0 = j * 32 + 4 * c0;
        auto factors = [&](int g, v4f& os, v4f& b) {
          if constexpr (HOIST_OS)
            os = hos[j][g];
          else
            os = *reinterpret_cast<const v4f*>(&cp_os[cl0 + 8 * g]);
          if constexpr (PLAIN)
            b = (v4f){0.f, 0.f, 0.f, 0.f};
          else if constexpr (HOIST_B)
            b = hb[j][g];
          else
            b = *reinterpret_cast<const v4f*>(&cp_b[cl0 + 8 * g]);
        };
        // all LDS reads of the fragment ahead of its arithmetic (the instantiations with fused
        // operators have no registers to spare for that and read as they go)
        constexpr bool kAhead = !POST && (!HOIST_OS || (!PLAIN && !HOIST_B));
        v4f os4[kAhead ? 4 : 1], b4[kAhead ? 4 : 1];
        if constexpr (kAhead) {
#pragma unroll
          for (int g = 0; g < 4; ++g) factors(g, os4[g], b4[g]);
          __builtin_amdgcn_sched_barrier(0);
        }
        uint32_t w[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          v4f os, b;
          if constexpr (kAhead) {
            os = os4[g];
            b = b4[g];
          } else {
            factors(g, os, b);
          }
          const ColParams c[4] = {{os[0], b[0], 0}, {os[1], b[1], 0}, {os[2], b[2], 0}, {os[3], b[3], 0}};
          w[g] = requant_pack4<EPI, PLAIN>(e, c, acc[j][4 * g + 0], acc[j][4 * g + 1],
                                           acc[j][4 * g + 2], acc[j][4 * g + 3]);
        }
        const auto s02 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
        const auto s13 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
        v4i v = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
        const int n = n0 + j * 32 + 16 * c0;
        // (operators fused behind the convolution: a table, or + residual [, ReLU] and quantize)
        if (POST && (e.table || e.resid_kind)) fused_tail16(e, tab, m, n, px_raw < p_end, v);
        if constexpr (STAGE) {
          // chunk c of tile row r in slot c ^ f(r), f such that the 16 lanes of a write phase
          // (16 consecutive rows, the same chunk) cover all banks
          const int r = lane & 31;
          const int slot = (2 * j + c0) ^ (NS == 64 ? (r >> 2) & 3 : (r >> 1) & (LPR - 1));
          *reinterpret_cast<v4i*>(stg + r * NS + slot * 16) = v;
        } else if (px_raw < p_end && n < e.N) {
          int8_t* dst = out + m * e.ldo + n;
          if (n + 15 < e.N) {
            *reinterpret_cast<v4i*>(dst) = v;
          } else {
#pragma unroll
            for (int t = 0; t < 16; ++t)
              if (n + t < e.N) dst[t] = (int8_t)((uint32_t)v[t >> 2] >> (8 * (t & 3)));
          }
        }
      });
    };
    if (plain)
      finish(IntC<1>());
    else
      finish(IntC<0>());
    if constexpr (STAGE) {
      // (the wave's own writes, in order: no barrier)
#pragma unroll
      for (int i = 0; i < NF; ++i) {
        const int u = i * 64 + lane;
        const int r = u / LPR;
        const int c = (u % LPR) ^ (NS == 64 ? (r >> 2) & 3 : (r >> 1) & (LPR - 1));
        const v4i v = *reinterpret_cast<const v4i*>(stg + u * 16);
        const int px2 = p0 + b * 32 + r;
        if (px2 < p_end && n0 + c * 16 < e.N)
          st_through(out + ((int64_t)img * hw + px2) * e.ldo + n0 + c * 16, v);
      }
    }
    DQ8_TRACE_WAVE(5 + 2 * ((b - wave) / NW));
  }
  DQ8_TRACE_POINT(3);
#else
  (void)p;
#endif
}

// ---- host side (qconv_direct.hip)
// Whether the streaming kernel can run the problem (stride and dilation 1 and a padding smaller
// than the filter are the caller's to check; here: a 3 x 3 or 1 x 1 filter on 64 or 128 input
// channels, sizes, and a tile whose patch fits the LDS next to the weights).  Chooses the pixel tile so that the workgroups come to whole rounds of the
// compute units with the least work per workgroup and fills tile_px, tiles_per_image, tiles_n,
// patch_bytes, in_bytes.
bool stream_conv_plan(DirectConvParams* p);
// whether the kernel is instantiated for a Kh x Kw filter on Ci channels
bool stream_conv_has_instance(int Kh, int Kw, int Ci);
int launch_stream_conv(int epilogue, const DirectConvParams& p, hipStream_t st);

}  // namespace dq8

#endif  // DQ8_QCONV_STREAM_H_
