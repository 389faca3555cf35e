// int8 GEMM for small M (a handful of tokens): the work is streaming W once, so the
// kernel is organised around memory parallelism, not MFMA utilisation.
//
//  * one workgroup per 16 output channels x (16 * MT) rows; N / 16 workgroups spread the
//    weight stream over the CUs;
//  * the K loop is split over the NW waves of the workgroup (wave w takes 64-deep
//    k-steps w, w + NW, ...) and every wave keeps U steps of loads in flight, so a
//    3072-deep reduction is 6 dependent steps instead of 48; partial sums meet in LDS;
//  * operands go straight from global memory into v_mfma_i32_16x16x64_i8 operand
//    layout (lane l: row l % 16, 16 k-bytes of group l / 16); W is the row operand, so
//    the 4 accumulator registers of a lane are 4 consecutive output channels.
// Needs K % 16 == 0 and 16-byte aligned, k-contiguous rows, like the other MFMA kernels.
#ifndef DQ8_QGEMM_SKINNY_H_
#define DQ8_QGEMM_SKINNY_H_

#include "q8_elementwise.h"
#include "qgemm_device.h"

namespace dq8 {

// U: k-steps a wave has in flight
template <int NW, int MT, int EPI, int U = 4>
__global__ void __launch_bounds__(NW * 64) qgemm_skinny_kernel(const MainParams p) {
  __shared__ int red[NW][MT][256];
  // per wave: one k-step of weights and of each row tile ([16 rows][64 k], 1 KiB each) on its
  // way from load order (consecutive lanes along a row) to fragment order
  __shared__ __attribute__((aligned(16))) int stage[NW][1 + MT][256];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int m0 = blockIdx.y * 16 * MT;
  const int KS = (p.K + 63) / 64;

  // Loads: lane l takes the 16-byte chunk l % 4 of row l / 4, so that four consecutive lanes
  // cover a 64-byte row segment (with every lane on a row of its own -- fragment order -- the
  // compute unit's address path served a load instruction as 64 separate accesses).
  const int lrow = lane >> 2, lchunk = lane & 3;
  const bool w_ok = n0 + lrow < p.N;
  const int8_t* wp = p.W + (int64_t)(w_ok ? n0 + lrow : p.N - 1) * p.ldw + lchunk * 16;
  const int8_t* ap[MT];
  bool a_ok[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    a_ok[t] = m0 + t * 16 + lrow < p.M;
    ap[t] = p.A + (int64_t)(a_ok[t] ? m0 + t * 16 + lrow : p.M - 1) * p.lda + lchunk * 16;
  }

  v4i acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (v4i){0, 0, 0, 0};

  const v4i zero = {0, 0, 0, 0};
  for (int ks0 = wave; ks0 < KS; ks0 += NW * U) {
    // unconditional loads (a branch around each would serialise them): a chunk past K
    // (K % 16 == 0: entirely inside or outside) or of a row past M / N is read from the
    // chunk's place in the first k-step instead and zeroed afterwards
    v4i wf[U], af[U][MT];
    bool in[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (ks0 + u * NW) * 64;
      in[u] = k + lchunk * 16 < p.K;
      const int kk = in[u] ? k : 0;
      wf[u] = *(const v4i*)(wp + kk);
#pragma unroll
      for (int t = 0; t < MT; ++t) af[u][t] = *(const v4i*)(ap[t] + kk);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // through the wave's own piece of LDS into fragment order: lane (r, g) wants chunk g of
      // row r, which lane 4 r + g loaded (LDS serves a wave's accesses in order: no barrier)
      *(v4i*)&stage[wave][0][lane * 4] = (in[u] && w_ok) ? wf[u] : zero;
#pragma unroll
      for (int t = 0; t < MT; ++t)
        *(v4i*)&stage[wave][1 + t][lane * 4] = (in[u] && a_ok[t]) ? af[u][t] : zero;
      const v4i wfrag = *(const v4i*)&stage[wave][0][r * 16 + g * 4];
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const v4i afrag = *(const v4i*)&stage[wave][1 + t][r * 16 + g * 4];
        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wfrag, afrag, acc[t], 0, 0, 0);
      }
    }
  }

  // D: register v of lane (r, g) is output channel 4g + v of row r
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][t][r * 16 + 4 * g + v] = acc[t][v];
  __syncthreads();

  for (int idx = threadIdx.x; idx < MT * 256; idx += NW * 64) {
    const int t = idx >> 8, e = idx & 255;
    const int m = m0 + t * 16 + (e >> 4), n = n0 + (e & 15);
    if (m >= p.M || n >= p.N) continue;
    int sum = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += red[w][t][e];
    const EpiParams& ep = p.epi;
    const ColParams c = col_params<EPI>(ep, n);
    const int64_t off = (int64_t)m * ep.ldo + n;
    if (EPI == DQ8_EPI_ACC_S32)
      ((int32_t*)ep.out)[off] = sum;
    else if (EPI == DQ8_EPI_DEQUANT_F32)
      ((float*)ep.out)[off] = finish_f32(ep, dequant_one_any(ep, c, sum, dequant_so(ep)), m, n);
    else
      ((int8_t*)ep.out)[off] = (int8_t)finish_s8(ep, requant_one<EPI>(ep, c, sum), m, n);
  }
}

// The same for f32 activations: mhlo_disc.quantize (per tensor, zero point 0, int8) runs on the
// activations on their way from memory into the MFMA operand registers, so that a quantized
// linear on a few dozen rows is one launch and the int8 activations never exist in memory.
// 16 rows x 16 output channels per workgroup (every workgroup along N quantizes its 16 rows
// again: the kernel is for a handful of row blocks, where that costs less than a launch).
// Both operands are loaded the way memory likes them -- consecutive lanes along a row: 16
// lanes per 256-byte row segment of the activations, 4 per 64-byte segment of the weights --
// and turned into MFMA fragments (a lane's 16 consecutive k of its row) through 1 KiB of LDS
// per wave and k-step that only that wave touches (no barrier).  With every lane fetching its
// own 64 bytes of its own row the compute unit's address path set the pace: 5.4 us per launch
// for 64 x 768 -> 768 against 7.9 us for quantize + GEMM; a branch around each load 9.2 us.
// The arithmetic is quant_one's, element for element (the division by the scale through its
// reciprocal, see div4_by_constant), so the result equals dq8_quantize followed by the int8
// kernel.
template <int NW, int EPI, int ROUND>
__global__ void __launch_bounds__(NW * 64) qgemm_skinny_f32a_kernel(const MainParams p) {
  constexpr int U = 2;  // k-steps in flight per wave
  __shared__ int red[NW][256];
  __shared__ __attribute__((aligned(16))) int xstage[NW][U][256];   // int8 [16 rows][64 k]
  __shared__ __attribute__((aligned(16))) int wstage[NW][U][256];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int m0 = blockIdx.y * 16;
  const int KS = (p.K + 63) / 64;

  // loads: activation instruction i covers rows 4 i .. 4 i + 3, lane l the 4 floats l % 16 of
  // row 4 i + l / 16; the weight instruction covers all 16 rows, lane l chunk l % 4 of row l / 4
  const int xrow = lane >> 4, xchunk = lane & 15;
  const int wrow = lane >> 2, wchunk = lane & 3;
  const float* xp[4];
  bool x_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + 4 * i + xrow;
    x_ok[i] = m < p.M;
    xp[i] = reinterpret_cast<const float*>(p.A) + (int64_t)(x_ok[i] ? m : p.M - 1) * p.lda;
  }
  const bool w_ok = n0 + wrow < p.N;
  const int8_t* wp = p.W + (int64_t)(w_ok ? n0 + wrow : p.N - 1) * p.ldw;
  const float s = p.a_scale[0];
  // (kernel-uniform) the division by the scale through its reciprocal, see div4_by_constant
  const float y = 1.0f / s;
  const bool fast = __builtin_fabsf(s) >= 0x1p-40f && __builtin_fabsf(s) <= 0x1p40f;

  // the output this thread finishes after the reduction, and its per-channel factors, fetched
  // now so that they arrive behind the operands instead of after the barrier
  const int e_m = m0 + ((threadIdx.x & 255) >> 4), e_n = n0 + (threadIdx.x & 15);
  const ColParams e_c = col_params<EPI>(p.epi, e_n < p.N ? e_n : p.N - 1);
  const float e_so = EPI == DQ8_EPI_DEQUANT_F32 ? dequant_so(p.epi) : 0.0f;

  v4i acc = {0, 0, 0, 0};
  const v4i zero = {0, 0, 0, 0};
  for (int ks0 = wave; ks0 < KS; ks0 += NW * U) {
    // Loads are unconditional (a branch around each would serialise them): a chunk past K
    // (K % 16 == 0: a chunk is entirely inside or outside), or of a row past M / N, is read
    // from the start of the (clamped) row instead and zeroed afterwards.
    v4i wq[U];
    float4 xq[U][4];
    bool xin[U], win[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (ks0 + u * NW) * 64;
      xin[u] = k + 4 * xchunk < p.K;
      win[u] = k + 16 * wchunk < p.K;
      wq[u] = *(const v4i*)(wp + (win[u] ? k + 16 * wchunk : 0));
#pragma unroll
      for (int i = 0; i < 4; ++i)
        xq[u][i] = *(const float4*)(xp[i] + (xin[u] ? k + 4 * xchunk : 0));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      using elementwise::pack4;
      using elementwise::quant_one;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 v = xq[u][i];
        int q;
        if (fast) {
          using elementwise::quant_from_quotient;
          const float4 t = elementwise::div4_by_constant(v, s, y);
          if constexpr (ROUND == 1)
            q = (int)elementwise::quant4_pack_rne(t);
          else
            q = (int)pack4(quant_from_quotient<ROUND>(t.x, -128.f, 127.f),
                           quant_from_quotient<ROUND>(t.y, -128.f, 127.f),
                           quant_from_quotient<ROUND>(t.z, -128.f, 127.f),
                           quant_from_quotient<ROUND>(t.w, -128.f, 127.f));
        } else {
          q = (int)pack4(quant_one<ROUND>(v.x, s, 0.f, -128.f, 127.f),
                         quant_one<ROUND>(v.y, s, 0.f, -128.f, 127.f),
                         quant_one<ROUND>(v.z, s, 0.f, -128.f, 127.f),
                         quant_one<ROUND>(v.w, s, 0.f, -128.f, 127.f));
        }
        xstage[wave][u][i * 64 + lane] = (xin[u] && x_ok[i]) ? q : 0;
      }
      *(v4i*)&wstage[wave][u][lane * 4] = (win[u] && w_ok) ? wq[u] : zero;
    }
    // (the same wave wrote what it reads: LDS serves a wave's accesses in order)
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const v4i af = *(const v4i*)&xstage[wave][u][r * 16 + g * 4];
      const v4i wf = *(const v4i*)&wstage[wave][u][r * 16 + g * 4];
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, af, acc, 0, 0, 0);
    }
  }

#pragma unroll
  for (int v = 0; v < 4; ++v) red[wave][r * 16 + 4 * g + v] = acc[v];
  __syncthreads();

  if (threadIdx.x < 256 && e_m < p.M && e_n < p.N) {
    const int e = threadIdx.x;
    int sum = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += red[w][e];
    const EpiParams& ep = p.epi;
    const int64_t off = (int64_t)e_m * ep.ldo + e_n;
    if (EPI == DQ8_EPI_ACC_S32)
      ((int32_t*)ep.out)[off] = sum;
    else if (EPI == DQ8_EPI_DEQUANT_F32)
      ((float*)ep.out)[off] = finish_f32(ep, dequant_one_any(ep, e_c, sum, e_so), e_m, e_n);
    else
      ((int8_t*)ep.out)[off] = (int8_t)finish_s8(ep, requant_one<EPI>(ep, e_c, sum), e_m, e_n);
  }
}

// One or two rows: a matrix times a vector or two.  One wave per output channel streams that
// channel's weight row from end to end -- 64 lanes x 16 bytes = 1 KiB contiguous per load
// instruction, U of them in flight -- and multiplies it with the activation rows, which the
// workgroup keeps in LDS, on the vector ALUs (v_dot4_i32_i8); the lanes' sums meet in a
// butterfly of cross-lane shuffles.  A row read linearly keeps one DRAM page open where 16
// rows read side by side keep 16, and every output channel is a wave of its own instead of a
// sixteenth of a workgroup.  Integer sums: the same bits as every other kernel.
// Needs K % 16 == 0, 16-byte aligned k-contiguous rows and MR * K bytes of LDS.
template <int NW, int MR, int U, int EPI>
__global__ void __launch_bounds__(NW * 64) qgemm_gemv_kernel(const MainParams p) {
  extern __shared__ __attribute__((aligned(16))) int8_t gemv_lds[];      // [MR][K]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * NW + __builtin_amdgcn_readfirstlane(wave);
  for (int i = threadIdx.x; i < MR * (p.K >> 4); i += NW * 64) {
    const int m = i / (p.K >> 4), k = (i - m * (p.K >> 4)) << 4;
    *(v4i*)(gemv_lds + m * p.K + k) =
        *(const v4i*)(p.A + (int64_t)(m < p.M ? m : p.M - 1) * p.lda + k);
  }
  __syncthreads();
  if (n >= p.N) return;                                    // (no barrier below)
  const int8_t* wp = p.W + (int64_t)n * p.ldw;
  int acc[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) acc[m] = 0;
  const v4i zero = {0, 0, 0, 0};
  for (int k0 = 16 * lane; k0 < p.K; k0 += U * 1024) {
    v4i wq[U];
#pragma unroll
    for (int u = 0; u < U; ++u) wq[u] = k0 + u * 1024 < p.K ? *(const v4i*)(wp + k0 + u * 1024) : zero;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u * 1024;
      if (k < p.K) {
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          const v4i a = *(const v4i*)(gemv_lds + m * p.K + k);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[m] = __builtin_amdgcn_sdot4(a[e], wq[u][e], acc[m], false);
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    int sum = acc[m];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0 && m < p.M) {
      const EpiParams& ep = p.epi;
      const ColParams c = col_params<EPI>(ep, n);
      const int64_t off = (int64_t)m * ep.ldo + n;
      if (EPI == DQ8_EPI_ACC_S32)
        ((int32_t*)ep.out)[off] = sum;
      else if (EPI == DQ8_EPI_DEQUANT_F32)
        ((float*)ep.out)[off] = finish_f32(ep, dequant_one_any(ep, c, sum, dequant_so(ep)), m, n);
      else
        ((int8_t*)ep.out)[off] = (int8_t)finish_s8(ep, requant_one<EPI>(ep, c, sum), m, n);
    }
  }
}

}  // namespace dq8

#endif  // DQ8_QGEMM_SKINNY_H_
