// Software-pipelined int8 MFMA GEMM for gfx950, used for the compute-bound
// (large M) regime.  Block tile BM x BN x 128, WM x WN waves, two LDS stages.
//
// What shapes this kernel is the CU's vector-memory front end, not the MFMA pipe: a
// 256x256 tile needs 64 KiB of operands per 128 of K, and the texture-address unit
// retires a 64-lane 16-byte load at a rate set by how many cache lines each group
// of four consecutive lanes touches.  Measured per CU (32 KiB, LDS-targeted loads):
// 16 rows x 64 B with consecutive lanes on different rows 2150 cycles; 8 rows x
// 128 B with consecutive lanes walking along a row 790 cycles; the 32 MFMAs that
// consume those bytes take about 1250.  Hence:
//  * BK = 128 and every load instruction covers 8 rows x one full 128-byte line,
//    lanes 8r .. 8r+7 on row r;
//  * loads write LDS directly (buffer_load_dwordx4 ... lds): no VGPR staging, no
//    ds_write, rows past M / N and bytes past the matrix arrive as zeros;
//  * a direct load puts lane i's 16 bytes at slot i of a 1 KiB block, so the block
//    is 8 rows x 128 B row-major in LDS.  Read back naively, the 32 rows of an MFMA
//    operand would hit the same banks; instead lane (r, s) fetches k-chunk
//    c = s ^ r ^ (block & 1) of its row, i.e. chunk c of row r lives in slot
//    c ^ r ^ (block & 1).  Any 8 consecutive rows then cover all 8 slots of a
//    128-byte bank row and any 16 cover both halves of a 256-byte one, so the
//    ds_read_b128 fragment reads are conflict free, while each quad of lanes still
//    reads one contiguous 64-byte segment of global memory;
//  * two 64 KiB stages fill the LDS.  All fragments of k-steps 2 and 3 are pulled
//    into registers during k-step 1, so a stage is dead from k-step 2 on: it is handed
//    back there ("stage free" barrier) and refilled while k-steps 2 and 3 still
//    compute from registers, two loads per row of four MFMAs.  A tile's loads thus get
//    most of a tile time to land before the "tile landed" barrier at k-step 3 of the
//    next tile.
// With random int8 operands and all 256 CUs busy the kernel is limited by the power
// the matrix cores draw, not by its schedule: the shader clock, 2.4 GHz when a few
// CUs run it, falls to 1.5-1.7 GHz (clock64 against wall_clock64), and variations of
// the schedule that change the cycle count leave the time per tile where it is.
// Waves per workgroup: the 256x256 tile runs on WM x WN = 2 x 4 waves, two per SIMD with a
// 128x64 wave tile.  Against 2 x 2 waves of 128x128 the requantisation of the epilogue -- a
// chain of VALU instructions of which a wave issues about one per 5 cycles -- is half as long
// per wave (5.7 -> 3.1 us), the accumulators fit ordinary VGPRs, and one wave's LDS and
// barrier waits are covered by the other's MFMAs.
// KSPLIT > 1: the workgroup has KSPLIT groups of WM x WN waves; group g runs the same
// pipeline, with LDS stages of its own, over k tiles [g * ceil(KT / KSPLIT), ...), and the
// groups' accumulators are added through LDS before group 0 runs the epilogue.  For
// problems with few output tiles and a deep K this puts KSPLIT times as many waves on the
// dependent chain of k tiles (a 3072-deep reduction on 64 x 64 tiles is 6 steps instead of
// 24) without a second kernel or global atomics.
// Requires K % 16 == 0 and 16-byte aligned, k-contiguous operands; the last k tile is
// completed with zeros (chunks at k >= K are given an out-of-range offset).
// CONV: the A operand is an NHWC image read in place as the im2col matrix (row m =
// (batch, ho, wo), k = (kh, kw, ci), Ci % 16 == 0); a lane recomputes the tap of its
// 16-byte chunk once per k tile, and taps that fall into the padding load zeros.
#ifndef DQ8_QGEMM_PIPELINED_H_
#define DQ8_QGEMM_PIPELINED_H_

#include <type_traits>

#include "qgemm_device.h"

// Timeline hook for profiling builds: a harness may define DQ8_TRACE_POINT(i) before
// including this header to record when a workgroup passes stage i (0 entry, 1 first
// tile landed, 2 main loop done, 3 results computed and stored).  Expands to nothing in
// the library.
#ifndef DQ8_TRACE_POINT
#define DQ8_TRACE_POINT(i)
#endif

namespace dq8 {

// gfx9 raw buffer descriptor word 3: 32-bit data format, no swizzle
constexpr int kBufferRsrcWord3 = 0x00020000;

typedef __attribute__((address_space(3))) void lds_void_t;

// 128-bit raw buffer descriptor (stride 0): base address, byte count, format word.  The
// descriptor is a scalar operand of the load: base and size are the same in every lane, and
// the readfirstlane says so where the compiler cannot see it (it folds away where it can).
__device__ __forceinline__ v4i make_rsrc(const void* base, int64_t num_records) {
  const uint64_t b = (uint64_t)base;
  v4i r = {__builtin_amdgcn_readfirstlane((int)(uint32_t)b),
           __builtin_amdgcn_readfirstlane((int)(uint32_t)((b >> 32) & 0xffff)),
           __builtin_amdgcn_readfirstlane((int)num_records), kBufferRsrcWord3};
  return r;
}

// One 16-byte-per-lane buffer load whose result goes straight to LDS: lane i's
// data lands at lds_addr + 16*i (lds_addr is wave-uniform and goes through M0).
// Issued as inline assembly so that the wave decides itself, with an explicit
// s_waitcnt vmcnt, when it needs the data; through the compiler builtin every LDS
// read would first wait for all loads in flight.
__device__ __forceinline__ void buffer_load_lds_b128(v4i rsrc, unsigned lds_addr, int voffset) {
  // (wave-uniform by construction; said explicitly for where the compiler cannot prove it)
  lds_addr = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_addr);
#pragma unroll
  for (int c = 0; c < 4; ++c) rsrc[c] = __builtin_amdgcn_readfirstlane(rsrc[c]);
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, 0 offen lds"
      :
      : "s"(lds_addr), "v"(voffset), "s"(rsrc)
      : "memory", "m0");
}

// s_waitcnt immediate for gfx9: vmcnt = n (6 bits, split), lgkmcnt = 0, expcnt = any
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4); }

// ROWMAP (with CONV false): the plain GEMM over the pixels a strided 1 x 1 filter reads.  Row m
// of A is input pixel (m / (Ho Wo), sh ((m / Wo) % Ho), sw_ (m % Wo)) of the NHWC image that H,
// Wd, Ci, Ho, Wo, sh, sw_ and conv_bytes describe (lda is not used): found once, before the k
// loop, which is the GEMM's -- half the instructions of the implicit GEMM's.
template <int BM, int BN, int WM, int WN, int KSPLIT, bool CONV, int EPI, bool ROWMAP = false>
__global__ void __launch_bounds__(WM* WN* KSPLIT * 64) qgemm_pipe_kernel(const MainParams p) {
  // The inline assembly only assembles in the device compilation; the host pass
  // just needs the kernel's stub.
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BK = 128;
  constexpr int NW = WM * WN;               // waves of one k group
  constexpr int NT = NW * KSPLIT * 64;      // threads of the workgroup
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int FM = TM / 32, FN = TN / 32;
  constexpr int NKS = BK / 32;              // MFMA k-steps per tile (4)
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  constexpr int STAGE = A_BYTES + B_BYTES;
  // one wave-wide load instruction moves one 8-row block: 8 rows x 128 B = 1 KiB
  constexpr int A_LD = (BM / 8) / NW;
  constexpr int B_LD = (BN / 8) / NW;
  constexpr int LD = A_LD + B_LD;           // load instructions per tile per wave
  static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0, "tile does not split over the waves");
  static_assert(FM >= 1 && FN >= 1, "fragment mismatch");
  static_assert(LD <= 63, "vmcnt is a 6-bit counter");
  static_assert(NW % 2 == 0, "the chunk a lane loads must not depend on the load slot");

  extern __shared__ __attribute__((aligned(1024))) int8_t smem_all[];
  DQ8_TRACE_POINT(0);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int kg = (tid >> 6) / NW;           // k group of this wave
  const int wave = (tid >> 6) % NW;         // wave index inside the group
  const int wm = wave / WN, wn = wave % WN;
  int8_t* smem = smem_all + kg * (2 * STAGE);

  int tm, tn;
  tile_coords(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int KT_ALL = (p.K + BK - 1) / BK;
  const int KT = (KT_ALL + KSPLIT - 1) / KSPLIT;   // k tiles per group
  const int kt0 = kg * KT;                          // first k tile of this group

  // ---- buffer descriptors over the rows this block may touch (GEMM) or the whole
  // image (convolution)
  constexpr int64_t kMaxRecords = 0x7fffffff;
  constexpr int kOutOfRange = (int)0x80000000;
  static_assert(!(CONV && ROWMAP), "rows mapped to pixels: a form of the plain GEMM");
  const int8_t* a_base = CONV || ROWMAP ? p.A : p.A + (int64_t)m0 * p.lda;
  const int8_t* w_base = p.W + (int64_t)n0 * p.ldw;
  const int64_t a_valid =
      CONV || ROWMAP ? p.conv_bytes : (int64_t)(p.M - m0 - 1) * p.lda + p.K;
  const int64_t w_valid = (int64_t)(p.N - n0 - 1) * p.ldw + p.K;
  const v4i a_rsrc = make_rsrc(a_base, a_valid < kMaxRecords ? a_valid : kMaxRecords);
  const v4i w_rsrc = make_rsrc(w_base, w_valid < kMaxRecords ? w_valid : kMaxRecords);
  // wave-uniform (it depends on the wave's k group only): keep it in a scalar register
  const unsigned lds_base =
      (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(size_t)(lds_void_t*)smem);

  // ---- load slots.  Instruction i of this wave covers 8-row block q = wave + i*NW;
  // lane -> row r = lane/8 of the block, LDS slot s = lane%8, global k-chunk
  // c = s ^ r ^ (q & 1).  NW is even, so q & 1 = wave & 1 and the lane loads the same
  // chunk c in every slot.
  const int lr = lane >> 3, ls = lane & 7;
  const int kc = (ls ^ lr ^ (wave & 1)) << 4;   // byte offset of the lane's chunk in a k tile
  int a_off[A_LD], b_off[B_LD];      // GEMM: byte offset of the lane's chunk in row 0 of the tile
  int a_lds[A_LD], b_lds[B_LD];      // wave-uniform LDS byte offset of the 1 KiB block
  // conv: the row's first input pixel (coordinates, and byte offset of its channel 0)
  int a_h[CONV ? A_LD : 1], a_w[CONV ? A_LD : 1], a_pix[CONV ? A_LD : 1];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int q = wave + i * NW;
    a_lds[i] = __builtin_amdgcn_readfirstlane(q * 1024);
    if (CONV) {
      const int m = m0 + q * 8 + lr;
      const int hw = p.Ho * p.Wo;
      const int n_img = m / hw, rem = m - n_img * hw;
      const int ho = rem / p.Wo, wo = rem - ho * p.Wo;
      // rows past M get a coordinate no tap can bring back into the image
      a_h[i] = m < p.M ? ho * p.sh - p.pad_t : -(1 << 24);
      a_w[i] = wo * p.sw_ - p.pad_l;
      a_pix[i] = m < p.M ? ((n_img * p.H + ho * p.sh - p.pad_t) * p.Wd + a_w[i]) * p.Ci : 0;
      a_off[i] = 0;
    } else if (ROWMAP) {
      // (rows past M read the last row again; their results are not stored)
      const int m = min(m0 + q * 8 + lr, p.M - 1);
      const int hw = p.Ho * p.Wo;
      const int n_img = m / hw, rem = m - n_img * hw;
      const int ho = rem / p.Wo, wo = rem - ho * p.Wo;
      a_off[i] = ((n_img * p.H + ho * p.sh) * p.Wd + wo * p.sw_) * p.Ci + kc;
    } else {
      a_off[i] = (q * 8 + lr) * (int)p.lda + kc;
    }
  }
#pragma unroll
  for (int i = 0; i < B_LD; ++i) {
    const int q = wave + i * NW;
    b_off[i] = (q * 8 + lr) * (int)p.ldw + kc;
    b_lds[i] = __builtin_amdgcn_readfirstlane(A_BYTES + q * 1024);
  }

  // Per k tile: is the lane's chunk inside K, and (conv) which tap does it belong to.
  // tile_setup(kt) precedes the issue_load calls of tile kt and is called with kt = 0, 1, 2, ...
  // in turn: the lane's chunk moves on by BK channels per call, i.e. by BK / Ci taps, BK % Ci
  // channels and at most one carry each from the channels into the taps and from the filter's
  // columns into its rows.  (Two integer divisions per call instead were a fifth of the VALU
  // instructions of a 64 x 64 tile's k loop, a hundred per k tile and wave next to four MFMAs;
  // such a tile's time is its wave's instruction count: 32 x 7 x 7 x 512, 3 x 3 -> 512: 12.7 ->
  // 11.5 us.)
  int t_koff = kOutOfRange, t_dh = 0, t_dw = 0, t_off = 0;
  int c_ci = 0, c_kh = 0, c_kw = 0;                  // the chunk's place in the filter, next call
  int d_ci = 0, d_kh = 0, d_kw = 0;                  // what BK channels add to it
  if (CONV) {
    const unsigned k = (unsigned)(kt0 * BK + kc);
    const unsigned tap = k / (unsigned)p.Ci;
    c_ci = (int)(k - tap * (unsigned)p.Ci);
    c_kh = (int)(tap / (unsigned)p.Kw);
    c_kw = (int)(tap - (unsigned)c_kh * (unsigned)p.Kw);
    const int d_tap = BK / p.Ci;
    d_ci = BK - d_tap * p.Ci;
    d_kh = d_tap / p.Kw;
    d_kw = d_tap - d_kh * p.Kw;
  }
  // (The same state kept per wave in scalar registers where Ci is a multiple of BK was measured
  // and is slower: a wave issues scalar and vector instructions from one stream, and the scalar
  // form has more of them.)
  auto tile_setup = [&](int kt) {
    const int k = (kt0 + kt) * BK + kc;
    const bool in = kt < KT && k < p.K;
    t_koff = in ? (kt0 + kt) * BK : kOutOfRange;
    if (CONV) {
      t_dh = c_kh * p.dh;
      t_dw = c_kw * p.dw;
      t_off = (t_dh * p.Wd + t_dw) * p.Ci + c_ci;
      c_ci += d_ci;
      const bool carry = c_ci >= p.Ci;
      c_ci -= carry ? p.Ci : 0;
      c_kw += d_kw + (carry ? 1 : 0);                  // (< 2 Kw)
      const bool wrap = c_kw >= p.Kw;
      c_kw -= wrap ? p.Kw : 0;
      c_kh += d_kh + (wrap ? 1 : 0);
    }
  };
  // issues load number `idx` (0 .. LD-1) of tile `kt` into stage `st`; chunks past the
  // end of K (and conv taps in the padding) get an out-of-range offset: zeros arrive,
  // no memory is touched
  auto issue_load = [&](int idx, int st) {
    const unsigned base = lds_base + st * STAGE;
#pragma unroll
    for (int i = 0; i < A_LD; ++i)
      if (i == idx) {
        int voff;
        if (CONV) {
          const int hi = a_h[i] + t_dh, wi = a_w[i] + t_dw;
          const bool ok = t_koff != kOutOfRange && (unsigned)hi < (unsigned)p.H &&
                          (unsigned)wi < (unsigned)p.Wd;
          voff = ok ? a_pix[i] + t_off : kOutOfRange;
        } else {
          // (t_koff out of range: 2^31 plus a row's offset, which the host keeps below 2^31, is
          // past every descriptor as well -- no select)
          voff = a_off[i] + t_koff;
        }
        buffer_load_lds_b128(a_rsrc, base + a_lds[i], voff);
      }
#pragma unroll
    for (int i = 0; i < B_LD; ++i)
      if (A_LD + i == idx)
        buffer_load_lds_b128(w_rsrc, base + b_lds[i],
                             b_off[i] + t_koff);
  };

  // ---- fragment addressing.  Operand row R = R0 + lane%32 sits in block R/8 at row
  // R%8; the k-chunk c = 2*ks + lane/32 of that row is in slot c ^ (R%8) ^ (block&1).
  // R0 is a multiple of 32, so the block parity is bit 3 of the lane.
  const int row_in_frag = lane & 31;
  const int swz = (lane & 7) ^ ((lane >> 3) & 1);
  int frag_off[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
    frag_off[ks] = (row_in_frag >> 3) * 1024 + (lane & 7) * 128 + (((2 * ks + (lane >> 5)) ^ swz) << 4);
  const int a_frag0 = (wm * TM / 8) * 1024;
  const int b_frag0 = A_BYTES + (wn * TN / 8) * 1024;

  // Four fragment sets, one per k-step of a tile.  Set ks+1 is read one step ahead;
  // during k-step 1 the sets for k-steps 2 AND 3 are read, so the stage is dead from
  // k-step 2 on.
  v4i fa[NKS][FM], fb[NKS][FN];
  auto load_frag_a = [&](int set, int st, int ks, int i) {
    fa[set][i] = *(const v4i*)(smem + st * STAGE + a_frag0 + i * 4096 + frag_off[ks]);
  };
  auto load_frag_b = [&](int set, int st, int ks, int j) {
    fb[set][j] = *(const v4i*)(smem + st * STAGE + b_frag0 + j * 4096 + frag_off[ks]);
  };

  v16i acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
  if (!CONV && __builtin_expect((p.corr_n != nullptr || p.corr_m != nullptr) && kg == 0, 0)) {
    // Zero points: sum (a - zx)(w - zw) = sum a w + corr_n[n] + corr_m[m]; starting the sums at
    // the corrections costs a few loads here and nothing in the epilogue, and int32
    // wraps the same way whichever end the terms are added at.  Element 4g+q of fragment
    // (i, j) is row i*32 + lane%32, column j*32 + 8g + 4(lane/32) + q of the wave tile.
    int cm[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = m0 + wm * TM + i * 32 + (lane & 31);
      cm[i] = p.corr_m ? p.corr_m[m < p.M ? m : p.M - 1] : 0;
    }
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * TN + j * 32 + 8 * g + 4 * (lane >> 5) + q;
          const int cn = p.corr_n ? p.corr_n[n < p.N ? n : p.N - 1] : 0;
#pragma unroll
          for (int i = 0; i < FM; ++i) acc[i][j][4 * g + q] = cn + cm[i];
        }
  }

  // Load schedule: the LD loads of tile t+2 are issued during k-steps 2 and 3 of tile
  // t, LPR per row of MFMAs, into the stage tile t has just released.
  static_assert(NKS == 4, "schedule below assumes four k-steps per tile");
  constexpr int LPR = (LD + 2 * FM - 1) / (2 * FM);          // loads per MFMA row
  constexpr int LD_KS2 = FM * LPR < LD ? FM * LPR : LD;       // loads issued during k-step 2

  // ---- prologue: all of tile 0, then all of tile 1.  The per-channel epilogue factors
  // are fetched behind tile 0: their cold loads and the division overlap its flight
  // instead of sitting between the main loop and the stores.  (Sending tile 1 out before
  // tile 0 has landed was measured and loses: every CU then pulls 128 KiB before the
  // first MFMA, and at full occupancy that start-up burst costs more than the one
  // exposed latency it saves.)
  tile_setup(0);
#pragma unroll
  for (int idx = 0; idx < LD; ++idx) issue_load(idx, 0);
  EarlyColParams<EPI, NT, BN> early;
  early.fetch(p.epi, n0);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  __syncthreads();
  DQ8_TRACE_POINT(1);
  tile_setup(1);
#pragma unroll
  for (int idx = 0; idx < LD; ++idx) issue_load(idx, 1);
#pragma unroll
  for (int i = 0; i < FM; ++i) load_frag_a(0, 0, 0, i);
#pragma unroll
  for (int j = 0; j < FN; ++j) load_frag_b(0, 0, 0, j);

  // One k tile out of stage `cur` (an int, or a compile-time constant: see below).
  auto k_tile = [&](auto cur_v, int kt) {
    const int cur = cur_v, nxt = cur ^ 1;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (ks == 2) {
        // this wave has read everything it needs from stage `cur`; once every wave
        // has, the stage can take tile kt+2
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
        __syncthreads();
        tile_setup(kt + 2);
      }
      if (ks == 3) {
        // tile kt+1 (older than the LD_KS2 loads of tile kt+2 just issued) has landed
        // for this wave; after the barrier, for all of them
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(LD_KS2));
        __syncthreads();
      }
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        // (row i of the MFMA grid also fetches the W fragments j = i, i + FM, ...)
        if (ks == 0) {
          load_frag_a(1, cur, 1, i);
#pragma unroll
          for (int j = i; j < FN; j += FM) load_frag_b(1, cur, 1, j);
        } else if (ks == 1) {
          load_frag_a(2, cur, 2, i);
#pragma unroll
          for (int j = i; j < FN; j += FM) load_frag_b(2, cur, 2, j);
          load_frag_a(3, cur, 3, i);
#pragma unroll
          for (int j = i; j < FN; j += FM) load_frag_b(3, cur, 3, j);
        } else if (ks == 2) {
#pragma unroll
          for (int l = 0; l < LPR; ++l) issue_load(i * LPR + l, cur);
        } else {
          load_frag_a(0, nxt, 0, i);
#pragma unroll
          for (int j = i; j < FN; j += FM) load_frag_b(0, nxt, 0, j);
#pragma unroll
          for (int l = 0; l < LPR; ++l) issue_load((FM + i) * LPR + l, cur);
        }
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks][j], fa[ks][i], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // The small tiles are a few MFMAs per k tile and wave, and their time is the wave's
  // instruction count: two k tiles per trip with the stage a constant turn the stage offsets of
  // the LDS reads and of the loads into immediate operands (a third of the vector instructions
  // of a 64 x 64 tile's k tile).
  constexpr bool kTwoPerTrip = BM * BN <= 128 * 128;
  if constexpr (kTwoPerTrip) {
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
      k_tile(std::integral_constant<int, 0>{}, kt);
      k_tile(std::integral_constant<int, 1>{}, kt + 1);
    }
    if (kt < KT) k_tile(std::integral_constant<int, 0>{}, kt);
  } else {
    for (int kt = 0; kt < KT; ++kt) k_tile(kt & 1, kt);
  }
  // nothing of this wave may still be writing LDS when the workgroup retires
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  DQ8_TRACE_POINT(2);

  if (KSPLIT > 1) {
    // add the groups' partial sums: groups 1.. park their accumulators in LDS (lane-major,
    // conflict free), group 0 collects them
    constexpr int PER_WAVE = FM * FN * 16 * 64;   // ints
    int* red = reinterpret_cast<int*>(smem_all);
    __syncthreads();   // every group is done with its operand stages
    if (kg > 0) {
      int* mine = red + ((kg - 1) * NW + wave) * PER_WAVE + lane;
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) mine[((i * FN + j) * 16 + v) * 64] = acc[i][j][v];
    }
    __syncthreads();
    if (kg == 0) {
#pragma unroll
      for (int g = 1; g < KSPLIT; ++g) {
        const int* theirs = red + ((g - 1) * NW + wave) * PER_WAVE + lane;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] += theirs[((i * FN + j) * 16 + v) * 64];
      }
    }
  }

  // (one k group: the whole workgroup takes part in the epilogue, and its LDS holds the block's
  // int8 tile behind the factors)
  constexpr bool kBlockStage = KSPLIT == 1 && (EPI == DQ8_EPI_REQUANT_CPU || EPI == DQ8_EPI_REQUANT_GPU) &&
                               BN * 12 + 512 + BM * BN <= 2 * STAGE;
  mfma_epilogue<EPI, FM, FN, NT, BN, NoHook, kBlockStage>(acc, p.epi, smem_all, m0 + wm * TM, n0 + wn * TN, n0,
                                                          early.c, wave, kg == 0);
  DQ8_TRACE_POINT(3);
#else
  (void)p;
#endif
}

}  // namespace dq8

#endif  // DQ8_QGEMM_PIPELINED_H_
