// Running minimum / maximum of a float tensor, per tensor or per channel: the statistic
// the calibration observers of the quantization tool accumulate before they derive scales
// and zero points.  HBM-bound: 4 bytes read per element, a few bytes written per workgroup.
//
// Two passes, no atomics, so the result does not depend on the order workgroups finish in
// and a NaN anywhere in a channel's data makes that channel's minimum and maximum NaN:
//   1. every workgroup reduces a slab of the tensor to one (min, max) pair per channel it
//      touches and writes it to the workspace;
//   2. a small second kernel reduces each channel's pairs and folds them into the running
//      values the caller keeps.
// The tensor is viewed as [outer, channels, inner], row-major.
//  * inner > 1 (or one channel): "rows" of `inner` contiguous elements, row r belongs to
//    channel r % channels; a workgroup reduces one segment of up to 4096 elements of one row
//    (16 bytes per thread per load, four loads in flight), one sweep over the tensor by many
//    small workgroups, as in the quantize kernels;
//  * inner == 1 and more than one channel (channel = last axis): threads along the channels,
//    four channels each, a workgroup walks a block of rows.
#include <algorithm>
#include <limits>
#include <mutex>

#include "dq8_common.h"
#include "disc_q8.h"

namespace dq8 {
namespace {

constexpr int kThreads = 256;
constexpr int kSegment = 4096;   // elements of one row a workgroup reduces (row kernel)

struct MinMax {
  float lo, hi;
};

// min / max that keep a NaN once they have seen one
__device__ __forceinline__ void fold(MinMax& m, float v) {
  m.lo = v < m.lo ? v : m.lo;
  m.hi = v > m.hi ? v : m.hi;
  if (v != v) {
    m.lo = v;
    m.hi = v;
  }
}
__device__ __forceinline__ void fold(MinMax& m, const MinMax& o) {
  const bool nan = o.lo != o.lo || m.lo != m.lo;
  m.lo = o.lo < m.lo ? o.lo : m.lo;
  m.hi = o.hi > m.hi ? o.hi : m.hi;
  if (nan) {
    m.lo = std::numeric_limits<float>::quiet_NaN();
    m.hi = m.lo;
  }
}

__device__ __forceinline__ MinMax identity() {
  return {std::numeric_limits<float>::infinity(), -std::numeric_limits<float>::infinity()};
}

// all-lanes reduction inside a wave, then over the waves of the workgroup through LDS;
// the result is valid in thread 0
__device__ __forceinline__ MinMax block_reduce(MinMax m) {
  __shared__ MinMax part[kThreads / 64];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    MinMax o;
    o.lo = __shfl_xor(m.lo, off, 64);
    o.hi = __shfl_xor(m.hi, off, 64);
    fold(m, o);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) part[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) fold(m, part[w]);
  }
  return m;
}

// ---- pass 1, rows: workgroup b reduces piece b % segs of row b / segs; a piece is `chunks`
// consecutive segments of kSegment elements (one segment unless the row is so long that the
// number of pairs per channel would make the second pass noticeable)
template <bool VEC>
__global__ void __launch_bounds__(kThreads)
minmax_rows(const float* __restrict__ x, int64_t inner, int segs, int chunks,
            float2* __restrict__ partial) {
  const int64_t row = blockIdx.x / segs;
  const int seg = (int)(blockIdx.x - row * segs);
  const float* p = x + row * inner;
  MinMax m = identity();
  for (int ch = 0; ch < chunks; ++ch) {
    const int64_t begin = ((int64_t)seg * chunks + ch) * kSegment;
    if (begin >= inner) break;
    const int64_t end = begin + kSegment < inner ? begin + kSegment : inner;
    if (VEC) {
      // row starts are 16-byte aligned: inner % 4 == 0 and an aligned tensor
      const float4* p4 = reinterpret_cast<const float4*>(p);
      const int64_t b4 = begin / 4, e4 = end / 4;
      float4 v[4];
      bool have[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t i = b4 + threadIdx.x + (int64_t)u * kThreads;
        have[u] = i < e4;
        if (have[u]) v[u] = p4[i];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (have[u]) {
          fold(m, v[u].x);
          fold(m, v[u].y);
          fold(m, v[u].z);
          fold(m, v[u].w);
        }
    } else {
      for (int64_t i = begin + threadIdx.x; i < end; i += kThreads) fold(m, p[i]);
    }
  }
  m = block_reduce(m);
  if (threadIdx.x == 0) partial[blockIdx.x] = make_float2(m.lo, m.hi);
}

// ---- pass 1, channel = last axis: x [rows, nch]; thread (tx, ty) of block (bx, by) owns
// channels 4 * (bx * blockDim.x + tx) .. + 3 and walks rows by * rows_per_block + ty,
// + blockDim.y, ...; partial[by][channel]
template <bool VEC>
__global__ void __launch_bounds__(kThreads)
minmax_lastaxis(const float* __restrict__ x, int64_t rows, int nch, int rows_per_block,
                float2* __restrict__ partial) {
  __shared__ MinMax stage[kThreads][4];
  constexpr int W = VEC ? 4 : 1;
  const int c0 = (blockIdx.x * blockDim.x + threadIdx.x) * W;
  const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end = r_begin + rows_per_block < rows ? r_begin + rows_per_block : rows;
  MinMax m[4] = {identity(), identity(), identity(), identity()};
  if (c0 < nch) {
    const int64_t step = blockDim.y;
    int64_t r = r_begin + threadIdx.y;
    if (VEC) {
      // eight rows' loads in flight per thread
      for (; r + 7 * step < r_end; r += 8 * step) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          v[u] = *reinterpret_cast<const float4*>(x + (r + u * step) * nch + c0);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          fold(m[0], v[u].x);
          fold(m[1], v[u].y);
          fold(m[2], v[u].z);
          fold(m[3], v[u].w);
        }
      }
      for (; r < r_end; r += step) {
        const float4 v = *reinterpret_cast<const float4*>(x + r * nch + c0);
        fold(m[0], v.x);
        fold(m[1], v.y);
        fold(m[2], v.z);
        fold(m[3], v.w);
      }
    } else {
      for (; r < r_end; r += step) fold(m[0], x[r * nch + c0]);
    }
  }
  // rows handled by the threadIdx.y > 0 slices fold into slice 0 through LDS
  const int t = threadIdx.y * blockDim.x + threadIdx.x;
#pragma unroll
  for (int k = 0; k < W; ++k) stage[t][k] = m[k];
  __syncthreads();
  if (threadIdx.y == 0 && c0 < nch) {
    for (int y = 1; y < (int)blockDim.y; ++y)
#pragma unroll
      for (int k = 0; k < W; ++k) fold(m[k], stage[y * blockDim.x + threadIdx.x][k]);
#pragma unroll
    for (int k = 0; k < W; ++k)
      if (c0 + k < nch) partial[(int64_t)blockIdx.y * nch + c0 + k] = make_float2(m[k].lo, m[k].hi);
  }
}

// ---- pass 2, rows layout: one workgroup per channel c; its pairs are
// partial[(o * channels + c) * segs + s], o < outer, s < segs
__global__ void __launch_bounds__(kThreads)
minmax_fold_rows(const float2* __restrict__ partial, int64_t outer, int channels, int segs,
                 float* __restrict__ min_io, float* __restrict__ max_io) {
  const int c = blockIdx.x;
  MinMax m = identity();
  for (int64_t o = 0; o < outer; ++o) {
    const float2* row = partial + (o * channels + c) * segs;
    int s = threadIdx.x;
    for (; s + 3 * kThreads < segs; s += 4 * kThreads) {      // four loads in flight
      const float2 v0 = row[s], v1 = row[s + kThreads], v2 = row[s + 2 * kThreads],
                   v3 = row[s + 3 * kThreads];
      fold(m, MinMax{v0.x, v0.y});
      fold(m, MinMax{v1.x, v1.y});
      fold(m, MinMax{v2.x, v2.y});
      fold(m, MinMax{v3.x, v3.y});
    }
    for (; s < segs; s += kThreads) {
      const float2 v = row[s];
      fold(m, MinMax{v.x, v.y});
    }
  }
  m = block_reduce(m);
  if (threadIdx.x == 0) {
    fold(m, MinMax{min_io[c], max_io[c]});
    min_io[c] = m.lo;
    max_io[c] = m.hi;
  }
}

// ---- pass 2, rows layout with few pairs per channel: one thread per channel
__global__ void __launch_bounds__(kThreads)
minmax_fold_rows_small(const float2* __restrict__ partial, int64_t outer, int channels, int segs,
                       float* __restrict__ min_io, float* __restrict__ max_io) {
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  MinMax m = identity();
  for (int64_t o = 0; o < outer; ++o)
    for (int s = 0; s < segs; ++s) {
      const float2 v = partial[(o * channels + c) * segs + s];
      fold(m, MinMax{v.x, v.y});
    }
  fold(m, MinMax{min_io[c], max_io[c]});
  min_io[c] = m.lo;
  max_io[c] = m.hi;
}

// ---- pass 2, last-axis layout: pairs partial[g * channels + c].  A workgroup takes 64
// channels; its four waves each reduce every fourth group and meet in LDS.
__global__ void __launch_bounds__(kThreads)
minmax_fold_lastaxis(const float2* __restrict__ partial, int groups, int channels,
                     float* __restrict__ min_io, float* __restrict__ max_io) {
  __shared__ MinMax part[kThreads];
  const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  MinMax m = identity();
  if (c < channels) {
    for (int g = slice; g < groups; g += kThreads / 64) {
      const float2 v = partial[(int64_t)g * channels + c];
      fold(m, MinMax{v.x, v.y});
    }
  }
  part[threadIdx.x] = m;
  __syncthreads();
  if (slice == 0 && c < channels) {
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) fold(m, part[w * 64 + lane]);
    fold(m, MinMax{min_io[c], max_io[c]});
    min_io[c] = m.lo;
    max_io[c] = m.hi;
  }
}

struct Plan {
  bool last_axis;
  int segs;             // rows layout: pieces per row
  int chunks;           // rows layout: segments per piece
  int64_t blocks;       // rows layout: workgroups of pass 1
  int bx, by, gx, gy, rows_per_block;   // last-axis layout
  int64_t pairs;        // (min, max) pairs in the workspace
};

bool make_plan(int64_t outer, int64_t channels, int64_t inner, bool vec, Plan* p) {
  *p = Plan{};
  if (inner == 1 && channels > 1) {
    p->last_axis = true;
    const int64_t units = vec ? channels / 4 : channels;
    int bx = 1;
    while (bx < kThreads && bx < units) bx *= 2;
    p->bx = bx;
    p->by = kThreads / bx;
    p->gx = (int)ceil_div(units, bx);
    // Row blocks: about 512 workgroups in all for the four-channels-per-thread form (eight
    // 16-byte loads in flight per thread), at least 64 rows each.  The same split is used for the one-channel-per-thread form, so
    // that the workspace does not depend on the alignment of the tensor.
    const int64_t units4 = ceil_div(channels, 4);
    const int64_t gx4 = ceil_div(units4, std::min<int64_t>(kThreads, units4));
    const int64_t gy_target = std::max<int64_t>(1, 512 / gx4);
    const int64_t rpb = std::max<int64_t>(ceil_div(outer, gy_target), 64);
    const int64_t gy = ceil_div(outer, rpb);
    if (gy > 65535 || rpb > (1 << 30)) return false;
    p->gy = (int)gy;
    p->rows_per_block = (int)rpb;
    p->pairs = gy * channels;
    return true;
  }
  const int64_t rows = outer * channels;
  // at most about 8192 pairs per channel, at most 64 segments per workgroup
  const int64_t all = ceil_div(inner, kSegment);
  const int64_t chunks = std::min<int64_t>(64, std::max<int64_t>(1, ceil_div(all * outer, 8192)));
  const int64_t segs = ceil_div(all, chunks);
  if (segs > (1 << 30) || rows * segs >= (1LL << 31)) return false;
  p->segs = (int)segs;
  p->chunks = (int)chunks;
  p->blocks = rows * segs;
  p->pairs = p->blocks;
  return true;
}

}  // namespace
}  // namespace dq8

using namespace dq8;

extern "C" size_t dq8_minmax_workspace_bytes(int64_t outer, int64_t channels, int64_t inner) {
  if (outer <= 0 || channels <= 0 || inner <= 0) return 0;
  Plan p;
  // (the space needed does not depend on whether the vectorised kernels can be used)
  if (!make_plan(outer, channels, inner, false, &p)) return 0;
  return (size_t)p.pairs * sizeof(float2);
}

namespace {

// Shared by the two entry points: both passes with the (min, max) pairs in `partial`.  Pass 1
// writes every pair pass 2 reads, so the scratch needs no particular contents beforehand.
int run_minmax(const float* x, int64_t outer, int64_t channels, int64_t inner,
               float* min_io, float* max_io, float2* partial, const Plan& p, bool vec,
               hipStream_t st) {
  if (p.last_axis) {
    const dim3 grid((unsigned)p.gx, (unsigned)p.gy), block((unsigned)p.bx, (unsigned)p.by);
    if (vec)
      hipLaunchKernelGGL(minmax_lastaxis<true>, grid, block, 0, st, x, outer, (int)channels,
                         p.rows_per_block, partial);
    else
      hipLaunchKernelGGL(minmax_lastaxis<false>, grid, block, 0, st, x, outer, (int)channels,
                         p.rows_per_block, partial);
    if (int s = check_hip(hipGetLastError(), "minmax_lastaxis launch")) return s;
    hipLaunchKernelGGL(minmax_fold_lastaxis, dim3((unsigned)ceil_div(channels, 64)),
                       dim3(kThreads), 0, st, partial, p.gy, (int)channels, min_io, max_io);
    return check_hip(hipGetLastError(), "minmax_fold_lastaxis launch");
  }
  if (vec)
    hipLaunchKernelGGL(minmax_rows<true>, dim3((unsigned)p.blocks), dim3(kThreads), 0, st, x,
                       inner, p.segs, p.chunks, partial);
  else
    hipLaunchKernelGGL(minmax_rows<false>, dim3((unsigned)p.blocks), dim3(kThreads), 0, st, x,
                       inner, p.segs, p.chunks, partial);
  if (int s = check_hip(hipGetLastError(), "minmax_rows launch")) return s;
  if (outer * p.segs <= 32 && channels >= 1024)
    hipLaunchKernelGGL(minmax_fold_rows_small, dim3((unsigned)ceil_div(channels, kThreads)),
                       dim3(kThreads), 0, st, partial, outer, (int)channels, p.segs, min_io, max_io);
  else
    hipLaunchKernelGGL(minmax_fold_rows, dim3((unsigned)channels), dim3(kThreads), 0, st, partial,
                       outer, (int)channels, p.segs, min_io, max_io);
  return check_hip(hipGetLastError(), "minmax_fold_rows launch");
}

}  // namespace

extern "C" int dq8_minmax(const float* x, int64_t outer, int64_t channels, int64_t inner,
                          float* min_io, float* max_io, void* workspace,
                          size_t workspace_bytes, void* stream) {
  clear_error();
  DQ8_REQUIRE(outer >= 0 && channels >= 0 && inner >= 0, "dq8_minmax: negative extent");
  if (outer == 0 || channels == 0 || inner == 0) return 0;   // nothing observed: state kept
  DQ8_REQUIRE(x && min_io && max_io, "dq8_minmax: null pointer");
  DQ8_REQUIRE(channels < (1LL << 31), "dq8_minmax: too many channels");
  const bool last_axis = inner == 1 && channels > 1;
  const bool vec = aligned(x, 16) && (last_axis ? channels % 4 == 0 : inner % 4 == 0);
  Plan p;
  DQ8_REQUIRE(make_plan(outer, channels, inner, vec, &p), "dq8_minmax: tensor too large");
  DQ8_REQUIRE(workspace && workspace_bytes >= (size_t)p.pairs * sizeof(float2),
              "dq8_minmax: workspace too small (see dq8_minmax_workspace_bytes)");
  return run_minmax(x, outer, channels, inner, min_io, max_io,
                    static_cast<float2*>(workspace), p, vec, (hipStream_t)stream);
}

// ---- the same with the pairs in memory the library brings along -------------------------
// For callers that cannot allocate (code under graph capture, serving loops that forbid
// hipMalloc): the (min, max) pairs of pass 1 live in a fixed array in device memory.  Every
// device the library runs on holds its own copy of the array at its own address, looked up
// once per device, with that device current, and kept; host code never uses the array's
// name for anything else.
namespace {

constexpr size_t kStaticScratchBytes = 4u << 20;   // 524288 (min, max) pairs
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the current device (nullptr + error status on failure)
int static_scratch(void** out) {
  int dev = 0;
  if (int s = check_hip(hipGetDevice(&dev), "hipGetDevice")) return s;
  DQ8_REQUIRE(dev >= 0 && dev < kMaxDevices, "dq8_minmax_static: device ordinal out of range");
  std::lock_guard<std::mutex> guard(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (int s = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)),
                          "hipGetSymbolAddress(scratch)"))
      return s;
    DQ8_REQUIRE(ptr != nullptr, "dq8_minmax_static: no device address for the scratch array");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

}  // namespace

extern "C" size_t dq8_minmax_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int dq8_minmax_static(const float* x, int64_t outer, int64_t channels, int64_t inner,
                                 float* min_io, float* max_io, void* stream) {
  clear_error();
  DQ8_REQUIRE(outer >= 0 && channels >= 0 && inner >= 0, "dq8_minmax_static: negative extent");
  if (outer == 0 || channels == 0 || inner == 0) return 0;
  DQ8_REQUIRE(x && min_io && max_io, "dq8_minmax_static: null pointer");
  DQ8_REQUIRE(channels < (1LL << 31), "dq8_minmax_static: too many channels");
  const bool last_axis = inner == 1 && channels > 1;
  const bool vec = aligned(x, 16) && (last_axis ? channels % 4 == 0 : inner % 4 == 0);
  Plan p;
  DQ8_REQUIRE(make_plan(outer, channels, inner, vec, &p), "dq8_minmax_static: tensor too large");
  DQ8_REQUIRE((size_t)p.pairs * sizeof(float2) <= kStaticScratchBytes,
              "dq8_minmax_static: this tensor needs " +
                  std::to_string((size_t)p.pairs * sizeof(float2)) +
                  " bytes of scratch, more than the built-in " +
                  std::to_string(kStaticScratchBytes) + "; use dq8_minmax with a workspace");
  void* ptr = nullptr;
  if (int s = static_scratch(&ptr)) return s;
  return run_minmax(x, outer, channels, inner, min_io, max_io,
                    static_cast<float2*>(ptr), p, vec, (hipStream_t)stream);
}
