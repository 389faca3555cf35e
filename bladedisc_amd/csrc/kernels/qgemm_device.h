// Device-side building blocks shared by the int8 GEMM and the implicit-GEMM
// convolution for gfx950: parameter blocks, the fused requantisation epilogue and
// the LDS-tiled MFMA main loop.
//
// Arithmetic contract of the epilogue (binary32, no contraction, IEEE division):
//   REQUANT_CPU  os = (sx*sw[n]) / (1*so);  d = (f32(acc) + b[n]) * os + zo
//                b[n] = f32(bias_s32[n])  or  f32(sat32(rne(bias_f32[n] * (1/(sx*sw[n])))))
//                (reference: ral/context/mkldnn/ideep/ideep/operators/matmul.hpp:532-535)
//   REQUANT_GPU  os = (sx[n]*sw[n]) / so[n];  d = os * f32(acc) + bias[n]
//                (reference: ral/context/quantized_gpu_kernel_impl.cc:262-265,385,416-420)
//   DEQUANT_F32  d = f32(acc) * (sx*sw[n]) + bias[n]
// followed, for the two requant modes, by saturation to [-128,127] and
// round-half-to-even.
#ifndef DQ8_QGEMM_DEVICE_H_
#define DQ8_QGEMM_DEVICE_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <utility>

#include "disc_q8.h"
#include "q8_elementwise.h"

#pragma clang fp contract(off)

// Timeline hook for profiling builds (see qgemm_pipelined.h): expands to nothing in the library.
#ifndef DQ8_TRACE_POINT
#define DQ8_TRACE_POINT(i)
#endif

namespace dq8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct EpiParams {
  void* out;
  int64_t ldo;  // elements
  int M, N;
  const void* bias;
  int bias_kind;
  const float* sx;
  const float* sw;
  const float* so;
  int sx_stride, sw_stride, so_stride;  // 0 (rank-0 scale) or 1 (per channel)
  int zo;
  // DEQUANT_F32 only.  0: out = f32(acc) * (sx sw) + bias.  1 / 2: the REQUANT_CPU /
  // REQUANT_GPU result q, dequantized in place: out = (float)(q - zo) * so[0].
  int requant;
  // REQUANT_CPU only.  1: the output stage is the integer one of the reference's AArch64
  // path -- (acc + bias) times a fixed-point multiplier and shift derived from
  // (sx sw[n]) / so, plus zo, clamped (see fixedpoint_one).
  int fixedpoint;
  // ---- operators fused behind the quantized result q (all optional; see disc_q8.h,
  // dq8_postops_t).  Residual: t = (float)(q - zo) * so[0] + r(m, n), then ReLU, then either
  // the f32 value is the output or it is quantized again: sat8(rne(t / out_scale + out_zp)).
  // Table: the int8 result indexes a 256-byte table.
  const void* resid;         // [M, N], row stride ldr elements; f32 or int8
  int64_t ldr;
  int resid_kind;            // 0 none, 1 f32, 2 int8 with (resid_scale[0], resid_zp)
  int resid_zp;
  const float* resid_scale;
  int relu;
  int out_zp;
  const float* out_scale;    // null: the residual form writes f32
  const uint8_t* table;
  int resid_vec;    // 1: residual rows may be read with aligned 16-byte loads
  int vec_store;    // 1: a group of 4 consecutive n may be stored as one 4/16-byte word
  int vec_store16;  // 1: int8 rows may be written with aligned 16-byte stores
};

// Operand description.  GEMM: A [M,K] (row stride lda), W [N,K] (row stride ldw).
// Convolution (NHWC x OHWI): GEMM row m = (batch, ho, wo), k = (kh, kw, ci).
struct MainParams {
  const int8_t* A;
  const int8_t* W;
  int64_t lda, ldw;
  int M, N, K;
  // convolution geometry (unused by the plain GEMM)
  int H, Wd, Ci, Ho, Wo, Kh, Kw;
  int pad_t, pad_l, sh, sw_, dh, dw;
  int64_t conv_bytes;   // size of the NHWC image tensor in bytes
  int tiles_m, tiles_n;
  // Zero-point corrections (pipelined GEMM kernels; null = none): the accumulator of
  // output (m, n) starts at corr_n[n] + corr_m[m] instead of 0.
  const int32_t* corr_n;
  const int32_t* corr_m;
  // f32 activations quantized on their way into the matrix cores (qgemm_skinny_f32a_kernel):
  // A then points to floats, lda counts floats, and a row is quantized per tensor with
  // a_scale[0] (device), zero point 0, to [-128, 127] with the given rounding
  const float* a_scale;
  int a_round_even;
  EpiParams epi;
};

// ------------------------------------------------------------------ epilogue
struct ColParams {  // per output channel
  float os;   // output scale (requant) or dequant scale
  float b;    // additive term, already in the units the mode needs
  int sh;     // fixed-point output stage only: the shift; os and b then hold the bit
              // patterns of the int32 multiplier and of the int32 bias
};

// ---- the integer output stage of the reference's AArch64 path
// (R ral/context/common_context_impl_quantization.cc:671-679, 865-872: Arm Compute Library's
// GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT; the library's published algorithm)
// saturating rounding doubling multiply, high half: (2 a b + 2^31) >> 32
__device__ __forceinline__ int sqrdmulh(int a, int b) {
  const long long t = (long long)a * (long long)b + (1ll << 30);
  const int r = (int)(t >> 31);
  return (a == (int)0x80000000 && b == (int)0x80000000) ? 0x7fffffff : r;
}
// x / 2^e, ties away from zero, e in [0, 31]
__device__ __forceinline__ int rounding_divide_by_pow2(int x, int e) {
  const int mask = (int)((1u << e) - 1u);
  const int threshold = (mask >> 1) + (x < 0 ? 1 : 0);
  return (x >> e) + ((x & mask) > threshold ? 1 : 0);
}
__device__ __forceinline__ int fixedpoint_one(int acc, int bias, int m0, int sh, int zo) {
  int v = (int)((unsigned)acc + (unsigned)bias);
  if (sh < 0) {
    const int left = -sh < 31 ? -sh : 31;
    v = sqrdmulh((int)((unsigned)v << left), m0);   // (the pre-multiplication wraps)
  } else {
    v = rounding_divide_by_pow2(sqrdmulh(v, m0), sh < 31 ? sh : 31);
  }
  v = (int)((unsigned)v + (unsigned)zo);
  return v < -128 ? -128 : (v > 127 ? 127 : v);
}
// multiplier = M0 2^-31 2^-shift with M0 in [2^30, 2^31): a binary32 has 24 significant bits,
// so q 2^31 below is an integer and the library's round() of it is the identity
__device__ __forceinline__ void fixedpoint_multiplier(float multiplier, int& m0, int& sh) {
  int e = 0;
  const float q = frexpf(multiplier, &e);
  m0 = (int)(q * 2147483648.0f);
  sh = -e;
}

__device__ __forceinline__ float sat_rne_s32_as_float(float v) {
  // saturate to int32 in float (the largest float below 2^31 is 2147483520), then
  // round to nearest even; the result is integral, so the later int->float
  // conversion of the stored s32 bias is the identity on it.
  v = fminf(fmaxf(v, -2147483648.0f), 2147483520.0f);
  return (float)(int)rintf(v);
}

// What col_params reads from memory for channel n, apart from the arithmetic on it: a kernel
// that wants the loads in flight early and the divisions late calls the two halves itself.
struct ColRaw {
  float sx, sw, so;
  int bias;   // the 32 bits of an f32 or s32 bias, an s8 bias sign-extended; 0 where none is read
};

template <int EPI>
__device__ __forceinline__ int col_mode(const EpiParams& p) {
  // the arithmetic the factors are for: a compile-time constant except under DEQUANT_F32
  return EPI != DQ8_EPI_DEQUANT_F32 ? EPI
         : p.requant == 1           ? DQ8_EPI_REQUANT_CPU
         : p.requant == 2           ? DQ8_EPI_REQUANT_GPU
                                    : DQ8_EPI_DEQUANT_F32;
}

template <int EPI>
__device__ __forceinline__ ColRaw col_fetch(const EpiParams& p, int n) {
  ColRaw r = {1.0f, 1.0f, 1.0f, 0};
  if (EPI == DQ8_EPI_ACC_S32) return r;
  r.sx = p.sx[(int64_t)n * p.sx_stride];
  r.sw = p.sw[(int64_t)n * p.sw_stride];
  const int mode = col_mode<EPI>(p);
  if (mode == DQ8_EPI_DEQUANT_F32) {
    if (p.bias_kind == DQ8_BIAS_F32) r.bias = ((const int32_t*)p.bias)[n];
    return r;
  }
  r.so = p.so[(int64_t)n * p.so_stride];
  if (mode == DQ8_EPI_REQUANT_CPU) {
    if (p.bias_kind == DQ8_BIAS_S32 || (!p.fixedpoint && p.bias_kind == DQ8_BIAS_F32))
      r.bias = ((const int32_t*)p.bias)[n];
  } else {  // REQUANT_GPU
    if (p.bias_kind == DQ8_BIAS_F32)
      r.bias = ((const int32_t*)p.bias)[n];
    else if (p.bias_kind == DQ8_BIAS_S8)
      r.bias = ((const int8_t*)p.bias)[n];
  }
  return r;
}

template <int EPI>
__device__ __forceinline__ ColParams col_finish(const EpiParams& p, const ColRaw& r) {
  ColParams c;
  c.os = 1.0f;
  c.b = 0.0f;
  c.sh = 0;
  if (EPI == DQ8_EPI_ACC_S32) return c;
  const float prod = r.sx * r.sw;
  const int mode = col_mode<EPI>(p);
  if (mode == DQ8_EPI_DEQUANT_F32) {
    c.os = prod;
    if (p.bias_kind == DQ8_BIAS_F32) c.b = __int_as_float(r.bias);
    return c;
  }
  const float so = r.so;
  if (mode == DQ8_EPI_REQUANT_CPU && p.fixedpoint) {
    int m0, sh;
    fixedpoint_multiplier(prod / so, m0, sh);
    c.os = __int_as_float(m0);
    c.sh = sh;
    c.b = __int_as_float(p.bias_kind == DQ8_BIAS_S32 ? r.bias : 0);
    return c;
  }
  if (mode == DQ8_EPI_REQUANT_CPU) {
    c.os = prod / (1.0f * so);
    if (p.bias_kind == DQ8_BIAS_S32) {
      c.b = (float)r.bias;
    } else if (p.bias_kind == DQ8_BIAS_F32) {
      const float bs = (1.0f * 1.0f) / prod;
      c.b = sat_rne_s32_as_float(__int_as_float(r.bias) * bs);
    }
  } else {  // REQUANT_GPU
    c.os = prod / so;
    if (p.bias_kind == DQ8_BIAS_F32)
      c.b = __int_as_float(r.bias);
    else if (p.bias_kind == DQ8_BIAS_S8)
      c.b = (float)r.bias;
  }
  return c;
}

template <int EPI>
__device__ __forceinline__ ColParams col_params(const EpiParams& p, int n) {
  return col_finish<EPI>(p, col_fetch<EPI>(p, n));
}

__device__ __forceinline__ int sat_rne_s8(float d) {
  d = fminf(fmaxf(d, -128.0f), 127.0f);  // NaN -> -128, like the CPU path
  return (int)rintf(d);
}

// int8 result of one accumulator for the two requant modes.  The additive terms are
// applied unconditionally (they are +0.0f when absent, which cannot change the
// rounded integer), so the per-element code has no branches.
template <int EPI>
__device__ __forceinline__ int requant_one(const EpiParams& p, const ColParams& c,
                                           int acc) {
  if (EPI == DQ8_EPI_REQUANT_CPU && p.fixedpoint)
    return fixedpoint_one(acc, __float_as_int(c.b), __float_as_int(c.os), c.sh, p.zo);
  float d = (float)acc;
  if (EPI == DQ8_EPI_REQUANT_CPU) {
    d = d + c.b;
    d = d * c.os;
    d = d + (float)p.zo;
  } else {
    d = c.os * d;
    d = d + c.b;
  }
  return sat_rne_s8(d);
}

// A 16-byte store that writes through the L2 (system scope: sc0 sc1).  An ordinary store leaves
// its line dirty in the L2 of the XCD that wrote it, and what is dirty when a kernel ends is
// written back before the next kernel starts -- about 1 us per 10 MB, after the last wave, under
// nothing.  Written through, the bytes leave while the kernel still runs.  Only for stores of
// which a wave instruction covers whole 64-byte pieces: 32-byte pieces written through take
// twice as long as ordinary ones.
__device__ __forceinline__ void st_through(void* p, const v4i& v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
#else
  *reinterpret_cast<v4i*>(p) = v;
#endif
}

// Four requantised results packed into one word (byte e = result of accumulator e).
// Same arithmetic as requant_one; rounding and conversion are done by adding
// 1.5 * 2^23: for |d| <= 128 the sum is rounded to an integer by the addition itself
// (round-to-nearest-even) and its low mantissa byte is the two's-complement int8.
//
// PLAIN: the launch has no bias and no output zero point, so the additive terms are +0.0f and
// are left out.  Adding +0.0f changes nothing but the sign of a zero, and a zero of either
// sign gives the byte 0 below, so the result is the same bit for bit.
template <int EPI, bool PLAIN = false>
__device__ __forceinline__ uint32_t requant_pack4(const EpiParams& p, const ColParams (&c)[4],
                                                  int a0, int a1, int a2, int a3) {
  const int acc[4] = {a0, a1, a2, a3};
  float clamped[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float d = (float)acc[e];
    if (EPI == DQ8_EPI_REQUANT_CPU) {
      if (!PLAIN) d = d + c[e].b;
      d = d * c[e].os;
      if (!PLAIN) d = d + (float)p.zo;
    } else {
      d = c[e].os * d;
      if (!PLAIN) d = d + c[e].b;
    }
    // v_med3_f32: one instruction for the clamp; with a NaN operand it returns the
    // minimum of the other two, so NaN -> -128 like the CPU path
    clamped[e] = __builtin_amdgcn_fmed3f(d, -128.0f, 127.0f);
  }
  // Rounding, conversion and packing in one instruction per result: adding 1.5 * 2^23 rounds
  // the clamped value to an integer (nearest even) and leaves its two's-complement int8 in
  // the low byte of the sum; the sub-dword form of the add (SDWA) writes exactly that byte
  // into byte e of the packed word and keeps the other bytes.
  const float magic = 12582912.0f;
  uint32_t word = __float_as_uint(clamped[0] + magic);   // byte 0; bytes 1 .. 3 are replaced below
#if defined(__HIP_DEVICE_COMPILE__)
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(word) : "v"(clamped[1]), "v"(magic));
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(word) : "v"(clamped[2]), "v"(magic));
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(word) : "v"(clamped[3]), "v"(magic));
#else
  word &= 0xffu;
  for (int e = 1; e < 4; ++e) word |= (__float_as_uint(clamped[e] + magic) & 0xffu) << (8 * e);
#endif
  return word;
}

// The output scale the fused requant -> dequantize forms multiply by (one load per kernel;
// unused otherwise).
__device__ __forceinline__ float dequant_so(const EpiParams& p) {
  return p.requant ? p.so[0] : 0.0f;
}

// ---- fused operators behind the quantized result (scalar forms; the hot paths below do the
// same arithmetic on vectors)
__device__ __forceinline__ float resid_at(const EpiParams& p, int64_t off) {
  if (p.resid_kind == 1) return ((const float*)p.resid)[off];
  return (float)((int)((const int8_t*)p.resid)[off] - p.resid_zp) * p.resid_scale[0];
}
// t = y + r, ReLU (a NaN stays a NaN)
__device__ __forceinline__ float resid_add(const EpiParams& p, float y, float r) {
  float t = y + r;
  if (p.relu) t = t < 0.0f ? 0.0f : t;
  return t;
}
// mhlo_disc.quantize to int8, round half to even: the arithmetic of dq8_quantize
__device__ __forceinline__ int quantize_s8(float t, float s, float z) {
  float v = t / s;
  v = v + z;
  v = rintf(v);
  v = fminf(fmaxf(v, -128.0f), 127.0f);
  return (int)v;
}
// the int8 that leaves the kernel for the stage's int8 result q; `roff` is the element's
// offset in the residual tensor
__device__ __forceinline__ int finish_s8_at(const EpiParams& p, int q, int64_t roff) {
  if (p.table) return (int)(int8_t)p.table[(uint8_t)q];
  if (p.resid_kind) {
    const float y = (float)(q - p.zo) * p.so[0];
    return quantize_s8(resid_add(p, y, resid_at(p, roff)), p.out_scale[0], (float)p.out_zp);
  }
  return q;
}
__device__ __forceinline__ int finish_s8(const EpiParams& p, int q, int64_t m, int n) {
  return finish_s8_at(p, q, m * p.ldr + n);
}
// the f32 that leaves the kernel for the dequantized stage result y
__device__ __forceinline__ float finish_f32_at(const EpiParams& p, float y, int64_t roff) {
  if (!p.resid_kind) return y;
  return resid_add(p, y, resid_at(p, roff));
}
__device__ __forceinline__ float finish_f32(const EpiParams& p, float y, int64_t m, int n) {
  return finish_f32_at(p, y, m * p.ldr + n);
}

// The four forms of the f32 epilogue.  Which one a launch runs is uniform over the kernel:
// the loops over the accumulators are instantiated per form (dispatch_f32_form) so that no
// per-element code tests it.
enum F32Form { kF32Plain = 0, kF32PlainBias = 1, kF32RequantCpu = 2, kF32RequantGpu = 3 };

__device__ __forceinline__ int f32_form(const EpiParams& p) {
  return p.requant ? 1 + p.requant : (p.bias_kind != DQ8_BIAS_NONE ? 1 : 0);
}

template <int FORM>
__device__ __forceinline__ float dequant_one(const EpiParams& p, const ColParams& c,
                                             int acc, float so_val) {
  if (FORM == kF32RequantCpu || FORM == kF32RequantGpu) {
    // requant_one's arithmetic, then dequantize's: (float)((int)q - zo) * so
    float d = (float)acc;
    if (FORM == kF32RequantCpu) {
      d = d + c.b;
      d = d * c.os;
      d = d + (float)p.zo;
    } else {
      d = c.os * d;
      d = d + c.b;
    }
    d = rintf(__builtin_amdgcn_fmed3f(d, -128.0f, 127.0f));
    // (added, not subtracted: a rounded -0.0 becomes the +0.0 that the integer
    // subtraction of dequantize yields)
    d = d + (float)(-p.zo);
    return d * so_val;
  }
  float d = (float)acc * c.os;
  if (FORM == kF32PlainBias) d = d + c.b;
  return d;
}

template <int V>
struct IntC {
  static constexpr int value = V;
};

// body(IntC<0>()), ..., body(IntC<N-1>()): a loop that is unrolled by construction, for code
// that indexes registers (an index the compiler does not see as a constant sends the whole
// array to scratch memory)
template <typename Body, int... I>
__device__ __forceinline__ void static_for_impl(Body&& body, std::integer_sequence<int, I...>) {
  (body(IntC<I>()), ...);
}
template <int N, typename Body>
__device__ __forceinline__ void static_for(Body&& body) {
  static_for_impl(body, std::make_integer_sequence<int, N>());
}

// body(IntC<form>) for the launch's form
template <typename Body>
__device__ __forceinline__ void dispatch_f32_form(const EpiParams& p, Body&& body) {
  switch (f32_form(p)) {
    case kF32Plain: body(IntC<kF32Plain>()); break;
    case kF32PlainBias: body(IntC<kF32PlainBias>()); break;
    case kF32RequantCpu: body(IntC<kF32RequantCpu>()); break;
    default: body(IntC<kF32RequantGpu>()); break;
  }
}

// one result, form looked up per call (the slow paths)
__device__ __forceinline__ float dequant_one_any(const EpiParams& p, const ColParams& c,
                                                 int acc, float so_val) {
  float r = 0.0f;
  dispatch_f32_form(p, [&](auto form) { r = dequant_one<decltype(form)::value>(p, c, acc, so_val); });
  return r;
}

// Stores the results for row m, columns n .. n+3 (n % 4 == 0).
template <int EPI>
__device__ __forceinline__ void store_group4(const EpiParams& p, int m, int n,
                                             const ColParams (&c)[4], int a0, int a1,
                                             int a2, int a3) {
  const int acc[4] = {a0, a1, a2, a3};
  const int64_t off = (int64_t)m * p.ldo + n;
  const bool full = n + 3 < p.N;
  if (EPI == DQ8_EPI_REQUANT_CPU || EPI == DQ8_EPI_REQUANT_GPU) {
    int8_t* out = (int8_t*)p.out;
    uint32_t w;
    // (launches with fused operators never come here: without 16-byte aligned output rows
    // they run on the generic kernel)
    if (EPI == DQ8_EPI_REQUANT_CPU && p.fixedpoint) {
      w = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        w |= ((uint32_t)requant_one<EPI>(p, c[e], acc[e]) & 0xffu) << (8 * e);
    } else {
      w = requant_pack4<EPI>(p, c, a0, a1, a2, a3);
    }
    if (full && p.vec_store) {
      *(uint32_t*)(out + off) = w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < p.N) out[off + e] = (int8_t)(w >> (8 * e));
    }
  } else if (EPI == DQ8_EPI_ACC_S32) {
    int32_t* out = (int32_t*)p.out;
    if (full && p.vec_store) {
      v4i w = {a0, a1, a2, a3};
      *(v4i*)(out + off) = w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < p.N) out[off + e] = acc[e];
    }
  } else {
    float* out = (float*)p.out;
    float f[4];
    const float so_val = dequant_so(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = dequant_one_any(p, c[e], acc[e], so_val);
    if (full && p.vec_store) {
      v4f w = {f[0], f[1], f[2], f[3]};
      *(v4f*)(out + off) = w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < p.N) out[off + e] = f[e];
    }
  }
}

// ----------------------------------------------------------------- main loop
// Workgroups are handed to the 8 XCDs round-robin and each XCD has its own L2, so
// each XCD gets a contiguous range of logical tiles, and logical tiles walk the tile
// grid in panels of kGroupM tile rows (column by column inside a panel).  The 32
// workgroups an XCD runs at a time then form a kGroupM x (32 / kGroupM) patch, which
// needs 4 + 8 operand row-blocks from beyond the L2 instead of the 2 + 16 of a
// row-major walk (measured at 4096^3: 144 MiB fetched by the L2s row-major, which is
// exactly 8 x 18 MiB).
constexpr int kGroupM = 4;

__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
  constexpr int kXcd = 8;
  if (nblocks % kXcd != 0) return bid;
  return (bid % kXcd) * (nblocks / kXcd) + bid / kXcd;
}

__device__ __forceinline__ void tile_coords(int bid, int nblocks, int tiles_m, int tiles_n,
                                            int& tm, int& tn) {
  const int t = xcd_remap(bid, nblocks);
  const int panel = t / (kGroupM * tiles_n);
  const int first_m = panel * kGroupM;
  const int rows = min(kGroupM, tiles_m - first_m);
  const int in_panel = t - panel * kGroupM * tiles_n;
  tm = first_m + in_panel % rows;
  tn = in_panel / rows;
}

// Operators fused behind the quantized result of an int8 epilogue.  `v` holds the 16 consecutive
// channels n .. n + 15 of output row m (which is also how the residual is read); `tab` is the
// 256-entry table in LDS when e.table is set; `row_ok`: the row exists.  Table:
// v = table[(uint8) v]; residual: v = quantize(resid_add(dequantize(v), r)) with the arithmetic
// of the separate library calls.
__device__ __forceinline__ void fused_tail16(const EpiParams& e, const uint8_t* tab, int64_t m,
                                             int n, bool row_ok, v4i& v) {
  if (e.table) {
    static_for<4>([&](auto dc) {
      constexpr int d = decltype(dc)::value;
      const uint32_t x = (uint32_t)v[d];
      v[d] = (int)((uint32_t)tab[x & 0xff] | ((uint32_t)tab[(x >> 8) & 0xff] << 8) |
                   ((uint32_t)tab[(x >> 16) & 0xff] << 16) | ((uint32_t)tab[x >> 24] << 24));
    });
  } else if (row_ok && n < e.N) {
    const float so_v = e.so[0], s2 = e.out_scale[0], z2 = (float)e.out_zp;
    const bool whole = e.resid_vec && n + 15 < e.N;
    const int64_t roff = m * e.ldr + n;
    // the residual of the 16 channels, as f32 (channels past N: unused zeros)
    v4f r[4];
    if (whole && e.resid_kind == 1) {
      const v4f* rp = reinterpret_cast<const v4f*>((const float*)e.resid + roff);
      static_for<4>([&](auto dc) { r[decltype(dc)::value] = rp[decltype(dc)::value]; });
    } else if (whole) {
      const float rs = e.resid_scale[0];
      const v4i rv = *reinterpret_cast<const v4i*>((const int8_t*)e.resid + roff);
      static_for<4>([&](auto dc) {
        constexpr int d = decltype(dc)::value;
        static_for<4>([&](auto bc) {
          constexpr int b = decltype(bc)::value;
          r[d][b] = (float)((int)(int8_t)((uint32_t)rv[d] >> (8 * b)) - e.resid_zp) * rs;
        });
      });
    } else {
      static_for<4>([&](auto dc) {
        constexpr int d = decltype(dc)::value;
        static_for<4>([&](auto bc) {
          constexpr int b = decltype(bc)::value;
          r[d][b] = n + 4 * d + b < e.N ? resid_at(e, roff + 4 * d + b) : 0.0f;
        });
      });
    }
    // The quantize that follows divides by the one scale of the launch: through its reciprocal
    // and two FMAs (the exact quotient, elementwise::div4_by_constant) and the clamp / round /
    // pack of dq8_quantize -- 13 instead of 28 vector instructions per result; a scale outside
    // the range that form is proved for takes the division.
    const float y2 = 1.0f / s2;
    const bool fast = elementwise::divisor_in_fast_range(s2);
    static_for<4>([&](auto dc) {
      constexpr int d = decltype(dc)::value;
      float t[4];
      static_for<4>([&](auto bc) {
        constexpr int b = decltype(bc)::value;
        const int q = (int)(int8_t)((uint32_t)v[d] >> (8 * b));
        t[b] = resid_add(e, (float)(q - e.zo) * so_v, r[d][b]);
      });
      if (fast) {
        float4 q4 = elementwise::div4_by_constant(make_float4(t[0], t[1], t[2], t[3]), s2, y2);
        q4.x = q4.x + z2;
        q4.y = q4.y + z2;
        q4.z = q4.z + z2;
        q4.w = q4.w + z2;
        v[d] = (int)elementwise::quant4_pack_rne(q4);
      } else {
        uint32_t w2 = 0;
        static_for<4>([&](auto bc) {
          constexpr int b = decltype(bc)::value;
          w2 |= ((uint32_t)quantize_s8(t[b], s2, z2) & 0xffu) << (8 * b);
        });
        v[d] = (int)w2;
      }
    });
  }
}

// Hook of mfma_epilogue: called once, after the int8 results have been computed into
// registers and before the first of them is stored (the default does nothing).
// kPostOps: whether the epilogue carries the code of the fused operators (residual, table) and
// of the fixed-point output stage; a kernel that is short of registers leaves them out and is
// not chosen for such launches.
struct NoHook {
  static constexpr bool kPostOps = true;
  __device__ __forceinline__ void operator()() const {}
};

template <int EPI, int FM, int FN, int NT, int BN, typename BeforeStores = NoHook, bool BLOCK_STAGE = false>
__device__ __forceinline__ void mfma_epilogue(v16i (&acc)[FM][FN], const EpiParams& e,
                                              int8_t* smem, int m_wave0, int n_wave0,
                                              int n_blk0, const ColParams* early = nullptr,
                                              int wave_slot = -1, bool active = true,
                                              int m_limit = -1, int8_t* stage_base = nullptr,
                                              BeforeStores before_stores = BeforeStores());

// The per-channel factors of the channels thread t is responsible for in the epilogue
// (t, t + NT, ...), fetched at the start of a kernel so that the cold loads of scales
// and bias and the division are off the critical path when the main loop ends.
template <int EPI, int NT, int BN>
struct EarlyColParams {
  static constexpr int kPerThread = (BN + NT - 1) / NT;
  ColParams c[kPerThread];
  __device__ __forceinline__ void fetch(const EpiParams& e, int n_blk0) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      // (a wave whose channels all lie past the block's BN has nothing to fetch)
      c[i] = ColParams{0.f, 0.f, 0};
      if ((int)(threadIdx.x & ~63u) + i * NT >= BN) continue;
      const int n = n_blk0 + (int)threadIdx.x + i * NT;
      c[i] = col_params<EPI>(e, n < e.N ? n : e.N - 1);
    }
  }
};

// LDS-tiled int8 GEMM on v_mfma_i32_32x32x32_i8.
//   block tile BM x BN x BK, WM x WN waves, each wave a (BM/WM) x (BN/WN) tile
//   built from 32x32 MFMA fragments; two LDS stages, global loads for stage
//   t+1 are in flight while stage t is multiplied.
// The weight rows are fed as the MFMA's row operand and the activation rows as
// its column operand, so each lane ends up with 4 consecutive output channels
// of one output row per accumulator quad: an aligned 4-byte (int8) or 16-byte
// (int32 / f32) store.
template <int BM, int BN, int BK, int WM, int WN, bool CONV, int EPI>
__global__ void __launch_bounds__(WM* WN * 64) qgemm_mfma_kernel(const MainParams p) {
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int FM = TM / 32, FN = TN / 32;
  constexpr int KC = BK / 16;        // 16-byte chunks per tile row
  constexpr int ROW = BK + 16;       // padded LDS row: conflict-free b128 reads
  constexpr int RPP = NT / KC;       // tile rows covered by one pass of the block
  constexpr int A_LD = BM / RPP, B_LD = BN / RPP;
  constexpr int STAGE = (BM + BN) * ROW;
  static_assert(BM % RPP == 0 && BN % RPP == 0, "tile/thread mismatch");
  static_assert(TM % 32 == 0 && TN % 32 == 0 && BK % 32 == 0, "fragment mismatch");

  extern __shared__ __attribute__((aligned(16))) int8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  int tm, tn;
  tile_coords(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  const int kc = tid % KC;
  const int lrow = tid / KC;

  // ---- per-thread global row descriptors (fixed for the whole K loop)
  const int8_t* a_ptr[A_LD];
  bool a_ok[A_LD];
  int a_hi0[A_LD], a_wi0[A_LD];  // conv only
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int m = m0 + lrow + i * RPP;
    a_ok[i] = m < p.M;
    const int mm = a_ok[i] ? m : 0;
    if (CONV) {
      const int hw = p.Ho * p.Wo;
      const int b = mm / hw;
      const int r = mm - b * hw;
      const int ho = r / p.Wo, wo = r - ho * p.Wo;
      a_hi0[i] = ho * p.sh - p.pad_t;
      a_wi0[i] = wo * p.sw_ - p.pad_l;
      a_ptr[i] = p.A + (int64_t)b * p.H * p.Wd * p.Ci;
    } else {
      a_hi0[i] = a_wi0[i] = 0;
      a_ptr[i] = p.A + (int64_t)mm * p.lda + kc * 16;
    }
  }
  const int8_t* b_ptr[B_LD];
  bool b_ok[B_LD];
#pragma unroll
  for (int i = 0; i < B_LD; ++i) {
    const int n = n0 + lrow + i * RPP;
    b_ok[i] = n < p.N;
    b_ptr[i] = p.W + (int64_t)(b_ok[i] ? n : 0) * p.ldw + kc * 16;
  }
  // conv: position of this thread's chunk inside the (kh, kw, ci) index space
  int c_ci = kc * 16, c_kw = 0, c_kh = 0;
  if (CONV) {
    while (c_ci >= p.Ci) {
      c_ci -= p.Ci;
      if (++c_kw == p.Kw) { c_kw = 0; ++c_kh; }
    }
  }

  v4i ra[A_LD], rb[B_LD];
  const v4i zero4 = {0, 0, 0, 0};

  auto gload = [&](int kt) {
    const bool k_ok = kt * BK + kc * 16 < p.K;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      if (CONV) {
        const int hi = a_hi0[i] + c_kh * p.dh, wi = a_wi0[i] + c_kw * p.dw;
        const bool ok = a_ok[i] && k_ok && hi >= 0 && hi < p.H && wi >= 0 && wi < p.Wd;
        const int8_t* src = a_ptr[i] + ((int64_t)(ok ? hi : 0) * p.Wd + (ok ? wi : 0)) * p.Ci + c_ci;
        ra[i] = ok ? *(const v4i*)src : zero4;
      } else {
        ra[i] = (a_ok[i] && k_ok) ? *(const v4i*)(a_ptr[i] + (int64_t)kt * BK) : zero4;
      }
    }
#pragma unroll
    for (int i = 0; i < B_LD; ++i)
      rb[i] = (b_ok[i] && k_ok) ? *(const v4i*)(b_ptr[i] + (int64_t)kt * BK) : zero4;
    if (CONV) {  // advance this thread's chunk by BK along k
      c_ci += BK;
      while (c_ci >= p.Ci) {
        c_ci -= p.Ci;
        if (++c_kw == p.Kw) { c_kw = 0; ++c_kh; }
      }
    }
  };
  auto lstore = [&](int buf) {
    int8_t* As = smem + buf * STAGE;
    int8_t* Bs = As + BM * ROW;
#pragma unroll
    for (int i = 0; i < A_LD; ++i)
      *(v4i*)(As + (lrow + i * RPP) * ROW + kc * 16) = ra[i];
#pragma unroll
    for (int i = 0; i < B_LD; ++i)
      *(v4i*)(Bs + (lrow + i * RPP) * ROW + kc * 16) = rb[i];
  };

  v16i acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  const int KT = (p.K + BK - 1) / BK;
  const int frag_off = (lane & 31) * ROW + (lane >> 5) * 16;

  if (KT > 0) {
    gload(0);
    lstore(0);
  }
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) gload(kt + 1);
    const int8_t* As = smem + buf * STAGE + (wm * TM) * ROW + frag_off;
    const int8_t* Bs = smem + buf * STAGE + BM * ROW + (wn * TN) * ROW + frag_off;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      v4i fa[FM], fb[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) fa[i] = *(const v4i*)(As + i * 32 * ROW + ks * 32);
#pragma unroll
      for (int j = 0; j < FN; ++j) fb[j] = *(const v4i*)(Bs + j * 32 * ROW + ks * 32);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) lstore(buf ^ 1);
    __syncthreads();
  }

  mfma_epilogue<EPI, FM, FN, NT, BN>(acc, p.epi, smem, m0 + wm * TM, n0 + wn * TN, n0);
}

// Epilogue shared by the MFMA kernels.  Accumulator v of fragment (i,j) belongs to
// output row m_wave0 + i*32 + lane%32 and channel n_wave0 + j*32 + 8*(v/4) +
// 4*(lane/32) + v%4.
//
// The per-channel factors are computed once per block (thread t -> channel t) and parked in
// LDS.  int8 results are packed four to a word, traded between the two halves of the wave so
// that a lane holds 16 consecutive channels of its row, and stored from the registers;
// int32 / f32 results are staged through LDS one fragment at a time so that they leave as
// full 128-byte row segments.
// BLOCK_STAGE (int8 results, every wave of the workgroup active, (NT / 64) wave tiles side by
// side covering the BN columns): results leave through LDS, behind the factors, in row order, with
// stores that write through the L2 (st_through; a lane pair's own 32-byte row pieces would be too
// small for those).  A wave tile of 64 channels stages and stores its own rows -- whole 64-byte
// pieces, no barrier; narrower or odd wave tiles are collected in one row-major tile of the
// whole block, and after a barrier the workgroup stores it BN bytes a row.  Measured, us per
// launch before / after: M = 6272, 256 -> 1024 7.65 / 7.0; M = 100352, 256 -> 128 13.0 / 11.7;
// M = 4096, 768 -> 3072 15.2 / 14.3; 4096^3 61.3 / 59.5.  The persistent kernels, whose epilogue
// holds its results in registers until the next tile's loads have landed, do the same per row
// of fragments where a wave tile is 64 channels wide (M = 16384, 768 -> 3072: 48.5 / 45.5); the
// block-wide form was measured there and lost (50.0 / 52.0: a barrier and an LDS trip per tile
// for results most of which are written long before the kernel ends).
template <int EPI, int FM, int FN, int NT, int BN, typename BeforeStores, bool BLOCK_STAGE>
__device__ __forceinline__ void mfma_epilogue(v16i (&acc)[FM][FN], const EpiParams& e,
                                              int8_t* smem, int m_wave0, int n_wave0,
                                              int n_blk0, const ColParams* early,
                                              int wave_slot, bool active, int m_limit,
                                              int8_t* stage_base, BeforeStores before_stores) {
  // `wave_slot`: which per-wave staging tile this wave uses (default: its index in the
  // workgroup); waves with `active` false only take part in the barriers; rows at or
  // past `m_limit` (default: M) are not stored; `stage_base`: where the per-wave staging
  // tiles start (default: right behind the per-channel factors at `smem`).
  const int m_end = m_limit >= 0 ? m_limit : e.M;
  constexpr int CP_BYTES = BN * 8;            // per-channel (scale, addend) pairs
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = wave_slot >= 0 ? wave_slot : tid >> 6;
  const int wn_off = n_wave0 - n_blk0;

  __syncthreads();  // every wave is done with the operand tiles
  float2* cp = reinterpret_cast<float2*>(smem);
  // (fixed-point output stage: the shifts, behind the pairs; that space is otherwise the
  // result staging of the 4-byte epilogues, which the stage does not use)
  int* cps = reinterpret_cast<int*>(smem + CP_BYTES);
  const bool fixedpoint = BeforeStores::kPostOps && EPI == DQ8_EPI_REQUANT_CPU && e.fixedpoint;
  if (early) {
#pragma unroll
    for (int i = 0; i < (BN + NT - 1) / NT; ++i) {
      const int t = tid + i * NT;
      if (t < BN) {
        cp[t] = make_float2(early[i].os, early[i].b);
        if (fixedpoint) cps[t] = early[i].sh;
      }
    }
  } else {
    for (int t = tid; t < BN; t += NT) {
      const int n = n_blk0 + t;
      const ColParams c = col_params<EPI>(e, n < e.N ? n : e.N - 1);
      cp[t] = make_float2(c.os, c.b);
      if (fixedpoint) cps[t] = c.sh;
    }
  }
  // (fused table lookup: the 256 bytes behind the shifts)
  uint8_t* tab = reinterpret_cast<uint8_t*>(smem + CP_BYTES + BN * 4);
  if (BeforeStores::kPostOps && e.table && tid < 64)
    reinterpret_cast<uint32_t*>(tab)[tid] = reinterpret_cast<const uint32_t*>(e.table)[tid];
  __syncthreads();
  DQ8_TRACE_POINT(5);
  if (!active) return;

  constexpr bool kInt8Out = EPI == DQ8_EPI_REQUANT_CPU || EPI == DQ8_EPI_REQUANT_GPU;
  if (kInt8Out && e.vec_store16) {
    // int8 results straight from the registers.  Of a 32 x 32 fragment a lane holds row
    // lane % 32 and the four channel quads 8 g + 4 (lane / 32) .. + 3, g = 0 .. 3, one packed
    // word each.  Two half-wave swaps (v_permlane32_swap) trade quads between lane l and
    // lane l + 32 so that the lower lane ends up with channels 0 .. 15 of its row and the
    // upper one with channels 16 .. 31: one 16-byte store per lane, 32 contiguous bytes per
    // row and instruction.  No LDS traffic (the first version staged the tile through LDS
    // with four-byte writes, eight to a bank).
    const bool plain = e.bias_kind == DQ8_BIAS_NONE && e.zo == 0;
    int8_t* out = static_cast<int8_t*>(e.out);
    // With a hook the results of the whole wave tile are formed first (32 registers per
    // 128 x 64), the hook runs, and the stores follow in one go; without one each fragment is
    // stored as soon as it is packed.
    constexpr bool kHook = !BLOCK_STAGE && !__is_same(BeforeStores, NoHook);
    v4i held[kHook ? FM : 1][kHook ? FN : 1];
    // block tile in LDS: chunk c (16 bytes) of row r in slot c ^ f(r % 32), f such that the 16
    // lanes of a write phase -- 16 consecutive rows, the same chunk -- cover all banks
    constexpr int kWN = BN / (FN * 32), kWM = (NT / 64) / kWN, kBM = kWM * FM * 32;
    constexpr int kChunks = BN / 16;
    auto swz = [](int r) {
      return BN % 256 == 0 ? (r & 15) : BN % 128 == 0 ? ((r >> 1) & 7) : ((r >> 2) & 3);
    };
    int8_t* tile = smem + CP_BYTES + BN * 4 + 256;
    const int row_wave0 = (wave / kWN) * (FM * 32);
    // With 64 channels to a wave tile a wave's own rows are whole 64-byte pieces: each wave
    // stages and stores its own tile, and the workgroup needs no barrier for it.
    constexpr bool kWavePrivate = FN == 2;
    auto store_frag = [&](const v4i v, int i, int j) {
      if constexpr (BLOCK_STAGE) {
        const int r = lane & 31;
        if constexpr (kWavePrivate) {
          // (a wave tile of 64 channels: rows of 64 bytes in the wave's own part of the area)
          *reinterpret_cast<v4i*>(tile + wave * (FM * 32 * 64) + (i * 32 + r) * 64 +
                                  (((2 * j + (lane >> 5)) ^ ((r >> 2) & 3)) << 4)) = v;
        } else {
          const int c = ((wn_off + j * 32) >> 4) + (lane >> 5);
          *reinterpret_cast<v4i*>(tile + (row_wave0 + i * 32 + r) * BN + ((c ^ swz(r)) << 4)) = v;
        }
        return;
      }
      const int n = n_wave0 + j * 32 + 16 * (lane >> 5);
      const int m = m_wave0 + i * 32 + (lane & 31);
      if (m < m_end && n < e.N) {
        int8_t* dst = out + (int64_t)m * e.ldo + n;
        if (n + 15 < e.N) {
          // (an ordinary store: the L2 merges the 32-byte pieces of a line; streamed past it,
          // non-temporal, the same stores take half as long again for the whole launch)
          *reinterpret_cast<v4i*>(dst) = v;
        } else {
#pragma unroll
          for (int b = 0; b < 16; ++b)
            if (n + b < e.N) dst[b] = (int8_t)((uint32_t)v[b >> 2] >> (8 * (b & 3)));
        }
      }
    };
    // MODE 0: float stage with its additive terms, 1: without them, 2: fixed-point stage
    auto store_all = [&](auto mode_c) {
      constexpr int MODE = decltype(mode_c)::value;
      // (static_for: with 16 fragments a loop this size is past what "#pragma unroll" unrolls,
      // and an accumulator array indexed by a loop variable lives in scratch memory)
      static_for<FN>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const int cl0 = wn_off + j * 32 + 4 * (lane >> 5);
        ColParams c[4][4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const v4f p01 = *reinterpret_cast<const v4f*>(&cp[cl0 + 8 * g]);
          const v4f p23 = *reinterpret_cast<const v4f*>(&cp[cl0 + 8 * g + 2]);
          v4i sh = {0, 0, 0, 0};
          if (MODE == 2) sh = *reinterpret_cast<const v4i*>(&cps[cl0 + 8 * g]);
          c[g][0] = {p01[0], p01[1], sh[0]};
          c[g][1] = {p01[2], p01[3], sh[1]};
          c[g][2] = {p23[0], p23[1], sh[2]};
          c[g][3] = {p23[2], p23[3], sh[3]};
        }
        static_for<FM>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          uint32_t w[4];
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            if (MODE == 2) {
              w[g] = 0;
#pragma unroll
              for (int q = 0; q < 4; ++q)
                w[g] |= ((uint32_t)fixedpoint_one(acc[i][j][4 * g + q], __float_as_int(c[g][q].b),
                                                  __float_as_int(c[g][q].os), c[g][q].sh, e.zo) &
                         0xffu)
                        << (8 * q);
            } else {
              w[g] = requant_pack4<EPI, MODE == 1>(e, c[g], acc[i][j][4 * g + 0], acc[i][j][4 * g + 1],
                                                   acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
            }
          }
          // swap(a, b): the upper half of a trades places with the lower half of b
          const auto s02 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
          const auto s13 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
          v4i v = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
          if (BeforeStores::kPostOps && (e.table || e.resid_kind)) {
            const int n = n_wave0 + j * 32 + 16 * (lane >> 5);
            const int64_t m = m_wave0 + i * 32 + (lane & 31);
            fused_tail16(e, tab, m, n, m < m_end, v);
          }
          if (kHook)
            held[kHook ? i : 0][kHook ? j : 0] = v;
          else
            store_frag(v, i, j);
        });
      });
    };
    if (fixedpoint)
      store_all(IntC<2>());
    else if (plain)
      store_all(IntC<1>());
    else
      store_all(IntC<0>());
    if (kHook) {
      before_stores();
      // A wave tile of 64 channels (the persistent 256 x 256 kernel): the 32 x 64 results of a
      // row of fragments go through the wave's own 4 KiB of staging (where the 4-byte epilogues
      // stage theirs) and leave as whole 64-byte row pieces, written through the L2 -- no
      // barrier, and nothing left dirty for the write-back after the last wave.
      constexpr bool kWaveStage = FN == 2;
      if constexpr (kWaveStage) {
        int8_t* stg = (stage_base ? stage_base : smem + CP_BYTES) + wave * 4096;
        static_for<FM>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          const int r = lane & 31;
#pragma unroll
          for (int j = 0; j < 2; ++j)
            *reinterpret_cast<v4i*>(stg + r * 64 + (((2 * j + (lane >> 5)) ^ ((r >> 2) & 3)) << 4)) =
                held[kHook ? i : 0][kHook ? j : 0];
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            const int u = k * 64 + lane;
            const int row = u >> 2;
            const int c = (u & 3) ^ ((row >> 2) & 3);
            const v4i v = *reinterpret_cast<const v4i*>(stg + u * 16);
            const int m = m_wave0 + i * 32 + row, n = n_wave0 + c * 16;
            if (m < m_end && n < e.N) {
              int8_t* dst = out + (int64_t)m * e.ldo + n;
              if (n + 15 < e.N) {
                st_through(dst, v);
              } else {
#pragma unroll
                for (int b = 0; b < 16; ++b)
                  if (n + b < e.N) dst[b] = (int8_t)((uint32_t)v[b >> 2] >> (8 * (b & 3)));
              }
            }
          }
        });
      } else {
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int i = 0; i < FM; ++i) store_frag(held[kHook ? i : 0][kHook ? j : 0], i, j);
      }
    }
    if constexpr (BLOCK_STAGE && kWavePrivate) {
      before_stores();
      const int8_t* mine = tile + wave * (FM * 32 * 64);
#pragma unroll
      for (int k = 0; k < FM * 2; ++k) {
        const int u = k * 64 + lane;
        const int row = u >> 2;
        const int c = (u & 3) ^ ((row >> 2) & 3);
        const int m = m_wave0 + row, n = n_wave0 + c * 16;
        if (m < m_end && n < e.N) {
          const v4i v = *reinterpret_cast<const v4i*>(mine + u * 16);
          int8_t* dst = out + (int64_t)m * e.ldo + n;
          if (n + 15 < e.N) {
            st_through(dst, v);
          } else {
#pragma unroll
            for (int b = 0; b < 16; ++b)
              if (n + b < e.N) dst[b] = (int8_t)((uint32_t)v[b >> 2] >> (8 * (b & 3)));
          }
        }
      }
    } else if constexpr (BLOCK_STAGE) {
      static_assert(kWM * kWN * 64 == NT && (kBM * kChunks) % NT == 0, "block tile over the workgroup");
      __syncthreads();
      before_stores();
      const int m_blk0 = m_wave0 - row_wave0;
#pragma unroll
      for (int k = 0; k < kBM * kChunks / NT; ++k) {
        const int u = tid + k * NT;
        const int row = u / kChunks;
        const int c = (u % kChunks) ^ swz(row & 31);
        const int m = m_blk0 + row, n = n_blk0 + c * 16;
        if (m < m_end && n < e.N) {
          const v4i v = *reinterpret_cast<const v4i*>(tile + u * 16);
          int8_t* dst = out + (int64_t)m * e.ldo + n;
          if (n + 15 < e.N) {
            st_through(dst, v);
          } else {
#pragma unroll
            for (int b = 0; b < 16; ++b)
              if (n + b < e.N) dst[b] = (int8_t)((uint32_t)v[b >> 2] >> (8 * (b & 3)));
          }
        }
      }
    }
    DQ8_TRACE_POINT(6);
    return;
  }
  before_stores();

  if (!kInt8Out && e.vec_store) {
    // int32 / f32 results: one 32 x 32 fragment (4 KiB) at a time through a per-wave LDS
    // tile, 128-byte rows with the 16-byte chunks swizzled by the row, then out as full
    // 128-byte row segments (8 lanes per row) instead of 32-byte pieces of 32 rows.
    int8_t* stage = (stage_base ? stage_base : smem + CP_BYTES) + wave * 4096;
    const float so_val = EPI == DQ8_EPI_DEQUANT_F32 ? dequant_so(e) : 0.0f;
    auto store_all = [&](auto form) {
    constexpr int FORM = decltype(form)::value;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int r = lane & 31;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int cl = wn_off + j * 32 + 8 * g + 4 * (lane >> 5);
          const int chunk = 2 * g + (lane >> 5);
          v4i w;
          if (EPI == DQ8_EPI_ACC_S32) {
            w = (v4i){acc[i][j][4 * g + 0], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                      acc[i][j][4 * g + 3]};
          } else {
            const v4f p01 = *reinterpret_cast<const v4f*>(&cp[cl]);
            const v4f p23 = *reinterpret_cast<const v4f*>(&cp[cl + 2]);
            const ColParams c[4] = {{p01[0], p01[1], 0}, {p01[2], p01[3], 0}, {p23[0], p23[1], 0}, {p23[2], p23[3], 0}};
#pragma unroll
            for (int q = 0; q < 4; ++q)
              w[q] = __float_as_int(dequant_one<FORM>(e, c[q], acc[i][j][4 * g + q], so_val));
          }
          *reinterpret_cast<v4i*>(stage + r * 128 + ((chunk ^ (r & 7)) << 4)) = w;
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int row = it * 8 + (lane >> 3), chunk = lane & 7;
          v4i v = *reinterpret_cast<const v4i*>(stage + row * 128 + ((chunk ^ (row & 7)) << 4));
          const int m = m_wave0 + i * 32 + row, n = n_wave0 + j * 32 + chunk * 4;
          if (m < m_end && n < e.N) {
            int32_t* dst = static_cast<int32_t*>(e.out) + (int64_t)m * e.ldo + n;
            if (BeforeStores::kPostOps && EPI == DQ8_EPI_DEQUANT_F32 && e.resid_kind) {
              // + residual (and ReLU) behind the dequantized result, read the way it is stored
              if (e.resid_vec && n + 3 < e.N) {
                float r[4];
                if (e.resid_kind == 1) {
                  const v4f rv = *reinterpret_cast<const v4f*>((const float*)e.resid + (int64_t)m * e.ldr + n);
#pragma unroll
                  for (int q = 0; q < 4; ++q) r[q] = rv[q];
                } else {
                  const float rs = e.resid_scale[0];
                  const uint32_t rw = *reinterpret_cast<const uint32_t*>((const int8_t*)e.resid + (int64_t)m * e.ldr + n);
#pragma unroll
                  for (int q = 0; q < 4; ++q) r[q] = (float)((int)(int8_t)(rw >> (8 * q)) - e.resid_zp) * rs;
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = __float_as_int(resid_add(e, __int_as_float(v[q]), r[q]));
              } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                  if (n + q < e.N) v[q] = __float_as_int(finish_f32(e, __int_as_float(v[q]), m, n + q));
              }
            }
            if (n + 3 < e.N) {
              st_through(dst, v);
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q)
                if (n + q < e.N) dst[q] = v[q];
            }
          }
        }
      }
    }
    };
    if (EPI == DQ8_EPI_DEQUANT_F32)
      dispatch_f32_form(e, store_all);
    else
      store_all(IntC<kF32Plain>());
    return;
  }

  // direct stores: 4 consecutive channels of one row per accumulator quad
  static_for<FN>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    static_for<4>([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      const int cl = wn_off + j * 32 + 8 * g + 4 * (lane >> 5);
      const int n = n_blk0 + cl;
      if (n >= e.N) return;
      const v4f p01 = *reinterpret_cast<const v4f*>(&cp[cl]);
      const v4f p23 = *reinterpret_cast<const v4f*>(&cp[cl + 2]);
      v4i sh = {0, 0, 0, 0};
      if (fixedpoint) sh = *reinterpret_cast<const v4i*>(&cps[cl]);
      const ColParams c[4] = {{p01[0], p01[1], sh[0]}, {p01[2], p01[3], sh[1]},
                              {p23[0], p23[1], sh[2]}, {p23[2], p23[3], sh[3]}};
      static_for<FM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const int m = m_wave0 + i * 32 + (lane & 31);
        if (m < m_end)
          store_group4<EPI>(e, m, n, c, acc[i][j][4 * g + 0], acc[i][j][4 * g + 1],
                            acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
      });
    });
  });
}

}  // namespace dq8

#endif  // DQ8_QGEMM_DEVICE_H_
