// Persistent form of the pipelined int8 MFMA GEMM (qgemm_pipelined.h) for problems with
// more output tiles than workgroup slots: a workgroup walks a list of tiles, and the first
// k tile of the NEXT output tile is sent for before the epilogue of the current one starts.
//
// Why: with one tile per workgroup and K of a few hundred (BERT's 768: six k tiles), the
// fixed parts of a tile are a third of its time -- about 1.7 us until the first k tile has
// landed, about 3 us of requantisation and stores, and between two rounds of workgroups the
// time the dispatcher needs to refill a compute unit.  Here the next tile's first loads fly
// while the VALU chain of the epilogue runs, and there is no refill.
//
// Differences from qgemm_pipe_kernel (same loads, LDS layout, fragment reads, schedule):
//  * k tile kt of every output tile uses stage (kt + 1) & 1, i.e. the first one lands in
//    stage 1, because stage 0 is where the epilogue of the previous tile stages its results;
//    the per-channel factors sit in stage 0 as well, behind that staging area;
//  * loads past the last k tile are not issued (their zeros could still be on their way into
//    the stage that the next tile's first loads target);
//  * tiles are dealt so that each XCD (workgroup index mod 8) keeps a contiguous range of
//    the panel-ordered tile list, as the one-tile kernels do.
#ifndef DQ8_QGEMM_PERSISTENT_H_
#define DQ8_QGEMM_PERSISTENT_H_

#include "qgemm_pipelined.h"

// Timeline hook for profiling builds: DQ8_TRACE_TILE(t, i) records when the workgroup passes
// stage i of tile t.  Expands to nothing in the library.
#ifndef DQ8_TRACE_TILE
#define DQ8_TRACE_TILE(t, i)
#endif

namespace dq8 {

// logical tile number `t` (panel order, see tile_coords) -> tile coordinates
__device__ __forceinline__ void panel_coords(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int panel = t / (kGroupM * tiles_n);
  const int first_m = panel * kGroupM;
  const int rows = min(kGroupM, tiles_m - first_m);
  const int in_panel = t - panel * kGroupM * tiles_n;
  tm = first_m + in_panel % rows;
  tn = in_panel / rows;
}

// Hook of the persistent kernel's epilogue: wait until this wave's loads have landed.
struct LoadsLanded {
  static constexpr bool kPostOps = false;   // (no registers to spare for the fused operators)
  __device__ __forceinline__ void operator()() const {
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  }
};

template <int BM, int BN, int WM, int WN, bool CONV, int EPI>
__global__ void __launch_bounds__(WM* WN * 64) qgemm_persist_kernel(const MainParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BK = 128;
  constexpr int NW = WM * WN;
  constexpr int NT = NW * 64;
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int FM = TM / 32, FN = TN / 32;
  constexpr int NKS = BK / 32;
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  constexpr int STAGE = A_BYTES + B_BYTES;
  constexpr int A_LD = (BM / 8) / NW;
  constexpr int B_LD = (BN / 8) / NW;
  constexpr int LD = A_LD + B_LD;
  static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0, "tile does not split over the waves");
  static_assert(FM >= 1 && FN >= 1, "fragment mismatch");
  static_assert(LD <= 63, "vmcnt is a 6-bit counter");
  static_assert(NW % 2 == 0, "the chunk a lane loads must not depend on the load slot");
  static_assert(NKS == 4, "schedule below assumes four k-steps per tile");
  static_assert(NW * 4096 <= STAGE, "the result staging of the 4-byte epilogues must fit stage 0");

  // Per-channel factors: in stage 0 behind the result staging of the 4-byte epilogues when
  // there is room (stage 0 holds no operands between the end of a main loop and the barrier
  // at the top of the next tile), else behind the two stages.
  constexpr int kCpInStage0 = NW * 4096 + BN * 12 + 256 <= STAGE;
  extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
  int8_t* const cp_smem = smem + (kCpInStage0 ? NW * 4096 : 2 * STAGE);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int KT = (p.K + BK - 1) / BK;
  DQ8_TRACE_TILE(blockIdx.x, 7);   // (workgroup b's first tile is not tile b in general: profiling only)

  // ---- the tiles of this workgroup: XCD x = blockIdx % 8 keeps tiles [x * per, (x+1) * per)
  // of the panel-ordered list when the counts divide, else a plain grid-stride walk
  const int total = p.tiles_m * p.tiles_n;
  const int grid = gridDim.x;
  constexpr int kXcd = 8;
  const bool by_xcd = total % kXcd == 0 && grid % kXcd == 0;
  const int t_first = by_xcd ? (blockIdx.x % kXcd) * (total / kXcd) + blockIdx.x / kXcd : blockIdx.x;
  const int t_step = by_xcd ? grid / kXcd : grid;
  const int t_end = by_xcd ? (blockIdx.x % kXcd + 1) * (total / kXcd) : total;

  constexpr int64_t kMaxRecords = 0x7fffffff;
  constexpr int kOutOfRange = (int)0x80000000;
  const unsigned lds_base =
      (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(size_t)(lds_void_t*)smem);

  // ---- load slots.  Instruction i of this wave covers 8-row block q = wave + i * NW; a
  // lane's byte offset is (its row in the block) * ld + (its k chunk), the same for every
  // block, plus the block's q * 8 * ld, which is wave-uniform and is added as a scalar.
  const int lr = lane >> 3, ls = lane & 7;
  const int kc = (ls ^ lr ^ (wave & 1)) << 4;
  const int a_lane = CONV ? 0 : lr * (int)p.lda + kc;
  const int b_lane = lr * (int)p.ldw + kc;
  int a_h[CONV ? A_LD : 1], a_w[CONV ? A_LD : 1], a_n[CONV ? A_LD : 1];
  auto a_lds = [&](int i) { return (wave + i * NW) * 1024; };
  auto b_lds = [&](int i) { return A_BYTES + (wave + i * NW) * 1024; };
  auto a_blk = [&](int i) { return (wave + i * NW) * 8 * (int)p.lda; };
  auto b_blk = [&](int i) { return (wave + i * NW) * 8 * (int)p.ldw; };

  // ---- state of the tile whose loads are being issued
  v4i a_rsrc = {0, 0, 0, kBufferRsrcWord3}, w_rsrc = {0, 0, 0, kBufferRsrcWord3};
  int m0 = 0, n0 = 0;
  auto enter_tile = [&](int t) {
    int tm, tn;
    panel_coords(t, p.tiles_m, p.tiles_n, tm, tn);
    // (workgroup-uniform: keep them, and the descriptors built from them, in scalar registers)
    m0 = __builtin_amdgcn_readfirstlane(tm * BM);
    n0 = __builtin_amdgcn_readfirstlane(tn * BN);
    const int8_t* a_base = CONV ? p.A : p.A + (int64_t)m0 * p.lda;
    const int8_t* w_base = p.W + (int64_t)n0 * p.ldw;
    const int64_t a_valid = CONV ? p.conv_bytes : (int64_t)(p.M - m0 - 1) * p.lda + p.K;
    const int64_t w_valid = (int64_t)(p.N - n0 - 1) * p.ldw + p.K;
    a_rsrc = make_rsrc(a_base, a_valid < kMaxRecords ? a_valid : kMaxRecords);
    w_rsrc = make_rsrc(w_base, w_valid < kMaxRecords ? w_valid : kMaxRecords);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      a_rsrc[c] = __builtin_amdgcn_readfirstlane(a_rsrc[c]);
      w_rsrc[c] = __builtin_amdgcn_readfirstlane(w_rsrc[c]);
    }
    if (CONV) {
#pragma unroll
      for (int i = 0; i < A_LD; ++i) {
        const int m = m0 + (wave + i * NW) * 8 + lr;
        const int hw = p.Ho * p.Wo;
        const int n_img = m / hw, rem = m - n_img * hw;
        const int ho = rem / p.Wo, wo = rem - ho * p.Wo;
        a_h[i] = m < p.M ? ho * p.sh - p.pad_t : -(1 << 24);
        a_w[i] = wo * p.sw_ - p.pad_l;
        a_n[i] = n_img * p.H * p.Wd;
      }
    }
  };

  // Per k tile: the lane's offsets for rows of block 0 (out of range, and staying so when
  // the block's scalar part is added, for chunks past K), and (conv) the tap of its chunk.
  int t_koff = kOutOfRange, t_abase = kOutOfRange, t_bbase = kOutOfRange, t_dh = 0, t_dw = 0, t_ci = 0;
  auto tile_setup = [&](int kt) {
    const int k = kt * BK + kc;
    const bool in = kt < KT && k < p.K;
    t_koff = in ? kt * BK : kOutOfRange;
    t_abase = in ? a_lane + kt * BK : kOutOfRange;
    t_bbase = in ? b_lane + kt * BK : kOutOfRange;
    if (CONV) {
      const unsigned tap = (unsigned)k / (unsigned)p.Ci;
      t_ci = k - (int)tap * p.Ci;
      const unsigned kh = tap / (unsigned)p.Kw;
      t_dh = (int)kh * p.dh;
      t_dw = (int)(tap - kh * p.Kw) * p.dw;
    }
  };
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
          voff = ok ? (a_n[i] + hi * p.Wd + wi) * p.Ci + t_ci : kOutOfRange;
        } else {
          voff = t_abase + a_blk(i);
        }
        buffer_load_lds_b128(a_rsrc, base + a_lds(i), voff);
      }
#pragma unroll
    for (int i = 0; i < B_LD; ++i)
      if (A_LD + i == idx) buffer_load_lds_b128(w_rsrc, base + b_lds(i), t_bbase + b_blk(i));
  };

  // ---- fragment addressing (see qgemm_pipelined.h)
  const int swz = (lane & 7) ^ ((lane >> 3) & 1);
  int frag_off[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
    frag_off[ks] = ((lane & 31) >> 3) * 1024 + (lane & 7) * 128 + (((2 * ks + (lane >> 5)) ^ swz) << 4);
  const int a_frag0 = (wm * TM / 8) * 1024;
  const int b_frag0 = A_BYTES + (wn * TN / 8) * 1024;
  v4i fa[NKS][FM], fb[NKS][FN];
  auto load_frag_a = [&](int set, int st, int ks, int i) {
    fa[set][i] = *(const v4i*)(smem + st * STAGE + a_frag0 + i * 4096 + frag_off[ks]);
  };
  auto load_frag_b = [&](int set, int st, int ks, int j) {
    fb[set][j] = *(const v4i*)(smem + st * STAGE + b_frag0 + j * 4096 + frag_off[ks]);
  };

  constexpr int LPR = (LD + 2 * FM - 1) / (2 * FM);
  constexpr int LD_KS2 = FM * LPR < LD ? FM * LPR : LD;

  // first tile of this workgroup: its first k tile is sent for here, every later tile's
  // before the epilogue of the tile in front of it
  EarlyColParams<EPI, NT, BN> early;
  if (t_first < t_end) {
    enter_tile(t_first);
    early.fetch(p.epi, n0);
    tile_setup(0);
#pragma unroll
    for (int idx = 0; idx < LD; ++idx) issue_load(idx, 1);
  }

  for (int t = t_first; t < t_end; t += t_step) {
    const int m0e = m0, n0e = n0;   // this tile's corner, kept for its epilogue
    DQ8_TRACE_TILE(t, 0);
    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    if (!CONV && __builtin_expect(p.corr_n != nullptr || p.corr_m != nullptr, 0)) {
      // zero points: the sums start at corr_n[n] + corr_m[m] (see qgemm_pipelined.h)
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

    // k tile 0 has landed in stage 1 for this wave (first tile: wait here; later tiles: the
    // epilogue of the previous tile waited before its stores, which may still be in flight);
    // after the barrier for every wave, and every wave is done with the result staging of
    // the previous tile in stage 0, which now takes k tile 1
    if (t == t_first)
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
    __syncthreads();
    DQ8_TRACE_TILE(t, 1);
    tile_setup(1);
    if (1 < KT) {
#pragma unroll
      for (int idx = 0; idx < LD; ++idx) issue_load(idx, 0);
    }
#pragma unroll
    for (int i = 0; i < FM; ++i) load_frag_a(0, 1, 0, i);
#pragma unroll
    for (int j = 0; j < FN; ++j) load_frag_b(0, 1, 0, j);

    for (int kt = 0; kt < KT; ++kt) {
      const int cur = (kt + 1) & 1, nxt = cur ^ 1;
      const bool more2 = kt + 2 < KT;   // (wave-uniform) is there a k tile to refill with
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        if (ks == 2) {
          __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
          __syncthreads();
          tile_setup(kt + 2);
        }
        if (ks == 3) {
          // k tile kt+1 has landed: it is older than the LD_KS2 loads of k tile kt+2 just
          // issued, if any were
          if (more2)
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(LD_KS2));
          else
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
          __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < FM; ++i) {
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
            if (more2) {
#pragma unroll
              for (int l = 0; l < LPR; ++l) issue_load(i * LPR + l, cur);
            }
          } else {
            load_frag_a(0, nxt, 0, i);
#pragma unroll
            for (int j = i; j < FN; j += FM) load_frag_b(0, nxt, 0, j);
            if (more2) {
#pragma unroll
              for (int l = 0; l < LPR; ++l) issue_load((FM + i) * LPR + l, cur);
            }
          }
#pragma unroll
          for (int j = 0; j < FN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks][j], fa[ks][i], acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    // every load of this wave has landed; every wave passed the last "stage free" barrier, so
    // nothing useful is read from either stage any more
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
    DQ8_TRACE_TILE(t, 2);

    // the next tile's per-channel factors and first k tile are sent for now and land
    // while this tile's results are requantised
    EarlyColParams<EPI, NT, BN> early_next = early;
    if (t + t_step < t_end) {
      enter_tile(t + t_step);
      early_next.fetch(p.epi, n0);
      tile_setup(0);
#pragma unroll
      for (int idx = 0; idx < LD; ++idx) issue_load(idx, 1);
    }

    // The epilogue forms its results, then waits until the loads just issued have landed
    // (they have had the whole requantisation to do so), then stores: the wait at the top of
    // the next tile therefore finds only stores in flight and does not wait for them (loads
    // and stores share the one counter).
    mfma_epilogue<EPI, FM, FN, NT, BN, LoadsLanded>(acc, p.epi, cp_smem, m0e + wm * TM,
                                                    n0e + wn * TN, n0e, early.c, wave, true, -1,
                                                    smem, LoadsLanded());
    early = early_next;
    DQ8_TRACE_TILE(t, 3);
  }
  // (the last iteration issued no loads after its final wait)
#else
  (void)p;
#endif
}

}  // namespace dq8

#endif  // DQ8_QGEMM_PERSISTENT_H_
