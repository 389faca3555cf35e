// A stand-in for one of the fused elementwise kernels the DISC compiler generates around a
// quantized GEMM and ships inside the compiled program as a code object: it dequantizes the
// GEMM's int8 result, applies ReLU and adds a residual.  Compiled to a gfx950 code object
// (hipcc --genco) by bladedisc_amd/build.py: build_test_code_objects(); the test program
// launches it through ral_kernel_launch.  All operations are single IEEE binary32
// operations, so a numpy float32 restatement reproduces it bit for bit.
#include <hip/hip_runtime.h>

#include <cstdint>

extern "C" __global__ void fused_dequant_relu_residual(const int8_t* q, const float* scale,
                                                       const float* residual, float* out,
                                                       int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float y = (float)q[i] * scale[0];
  out[i] = (y > 0.0f ? y : 0.0f) + residual[i];
}
