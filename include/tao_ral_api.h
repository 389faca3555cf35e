/*
 * tao_ral_api.h -- the runtime-plugin C ABI that code compiled by the DISC compiler
 * (and the TorchBlade / TF bridges) binds to, implemented for one MI355X.
 *
 * The first three functions and kMlirLoweredEntry are the reference's own ABI
 * (R = alibaba/BladeDISC tao_compiler/mlir/ral/ral_api.h:37-67, ral_api.cc:29-51):
 * a compiled program's `main` receives {ExecutionContext*, &tao_ral_call_impl} and
 * calls every runtime service as
 *     tao_ral_call_impl(exec_ctx, "<name>___<device>___<arg codes>___<ret codes>", args)
 * with `args` packed as R disc/transforms/disc_to_llvm.cc:302-365 packs them.
 *
 * The disc_ral_* functions are a C view of what the reference exposes only as C++
 * (MakeBaseCudaContext, R ral/context/base/cuda/cuda_context_impl.cc:168-202, and
 * the BaseCudaExecutionContext constructor), so that hosts without a C++ binding
 * (ctypes, cgo, JNI) can create the contexts the calls above need.
 *
 * Entries registered for the gpu device (query with disc_ral_api_name):
 *   ral_qgemm, ral_pdll_qgemm, ral_pdll_qgemm_per_channel, ral_qconv,
 *   ral_quantize, ral_dequantize, and the driver set alloc, dealloc,
 *   ral_gpu_alloc_persistent, raw_gpu_alloc, raw_gpu_dealloc, h2d_, d2h_, d2d_,
 *   ral_gpu_memset, ral_gpu_get_stream, sync_on_stream, ral_gpu_sync_all,
 *   ral_gpu_as_cu_stream, ral_gpu_as_se_stream, ral_kernel_launch.
 */
#ifndef TAO_RAL_API_H_
#define TAO_RAL_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* name of the entry function of a compiled program: "main" */
extern const char* const kMlirLoweredEntry;

typedef void* tao_ral_context_t;
typedef int32_t tao_ral_status_t; /* 0 = ok */

/* Calls the registered function `name` (a NUL-terminated const char*).  `ctx` is an
 * ExecutionContext handle.  An unknown name puts the context into error state. */
void tao_ral_call_impl(tao_ral_context_t ctx, void* name, void** args);

/* Status of a Context handle since the last clear; *err_msg (if not NULL) points at
 * a thread-local copy of the message, empty when ok. */
tao_ral_status_t tao_ral_last_error(tao_ral_context_t ctx, const char** err_msg);

/* Leaves error state.  `ctx` is a Context handle. */
void tao_ral_clear_error(tao_ral_context_t ctx);

/* ---- context lifetime -------------------------------------------------- */

typedef void* (*disc_ral_alloc_fn)(size_t bytes, void* user);
typedef void (*disc_ral_dealloc_fn)(void* ptr, void* user);

/* Creates a Context for the current HIP device.  All copies and launches issued
 * through it go to `hip_stream` (a hipStream_t; NULL = the null stream).  When
 * `alloc`/`dealloc` are given, device memory comes from them (e.g. the embedding
 * framework's caching allocator); otherwise from hipMalloc behind a size-class pool.
 * `cache_workspace` != 0 keeps freed pool memory across executions.  Returns NULL on
 * failure. */
tao_ral_context_t disc_ral_context_create(void* hip_stream, int device_ordinal,
                                          disc_ral_alloc_fn alloc,
                                          disc_ral_dealloc_fn dealloc, void* user,
                                          int cache_workspace);
/* Same, for running a whole compiled program: `metadata_file_path` names the program's
 * constant store (the side file the compiler writes, ral/ral_metadata.cc:60-200), from
 * which ral_const serves constants by name; NULL = no constants.  Counterpart of
 * BaseContextOption::metadata_file_path (context/base/base_context.h:29-34). */
tao_ral_context_t disc_ral_context_create_for_program(void* hip_stream, int device_ordinal,
                                                      disc_ral_alloc_fn alloc,
                                                      disc_ral_dealloc_fn dealloc, void* user,
                                                      int cache_workspace,
                                                      const char* metadata_file_path);
void disc_ral_context_destroy(tao_ral_context_t ctx);

/* One ExecutionContext per run of a compiled program; destroying it returns every
 * buffer the run allocated and did not hand back. */
tao_ral_context_t disc_ral_execution_context_create(tao_ral_context_t ctx);
void disc_ral_execution_context_destroy(tao_ral_context_t exec_ctx);
tao_ral_context_t disc_ral_execution_context_get_context(tao_ral_context_t exec_ctx);

/* Program inputs and outputs: C face of ExecutionContext::bindInput / bindOutput
 * (ral/ral_context.h:164-167; context/base/base_context.cc:63-95).  Inputs are borrowed.
 * An output handle owns its buffer when the program allocated it and nothing else
 * refers to it (disc_ral_output_owned): destroying the handle then returns the buffer to
 * the context's allocator, unless disc_ral_output_release was called first, which
 * leaves the buffer to the caller.  Outputs that alias an input or a constant are never
 * freed by the handle.  bind_input returns 0 on success. */
typedef void* disc_ral_output_t;
int disc_ral_execution_bind_input(tao_ral_context_t exec_ctx, int input_idx, void* buffer,
                                  const int64_t* shape, int rank);
disc_ral_output_t disc_ral_execution_take_output(tao_ral_context_t exec_ctx, int output_idx);
const void* disc_ral_output_data(disc_ral_output_t output);
int disc_ral_output_rank(disc_ral_output_t output);
int64_t disc_ral_output_dim(disc_ral_output_t output, int i);
int disc_ral_output_owned(disc_ral_output_t output);
void disc_ral_output_release(disc_ral_output_t output);
void disc_ral_output_destroy(disc_ral_output_t output);

/* Writes / inspects a constant store in the reference's metadata-file format
 * (ral/ral_metadata.cc:60-200): names[i] -> hex_values[i] (the constant's bytes as a
 * hexadecimal string), a host constant where is_host[i] != 0, else a device constant.
 * A constant's name is "<id>_<element type>_<d0xd1...>", e.g. "w0_i8_768x768".
 * disc_ral_metadata_count loads a file and counts how many of the probe names it holds
 * as host and as device constants.  Both return 0 on success.  Host only. */
int disc_ral_metadata_emit(const char* path, int count, const uint8_t* is_host,
                           const char* const* names, const char* const* hex_values);
int disc_ral_metadata_count(const char* path, int* host_constants, int* device_constants,
                            const char* const* probe_names, int n_probe);

/* ---- registry introspection ------------------------------------------- */

int disc_ral_api_count(void);
/* index in [0, count): keys in sorted order (full mangled names and bare names) */
const char* disc_ral_api_name(int index);
int disc_ral_api_exists(const char* name);

/* Diagnostic: what ral_pdll_qconv2d derives from its TensorFlow-style attributes
 * (the rules of tao_compiler/mlir/ral/context/common_context_impl_quantization.h:27-206):
 * padding {lo0,hi0,lo1,hi1}, the 17-entry ral_qconv metadata vector and the result
 * shape.  Weights are [out_channels, filter_h, filter_w, in_channels].  Returns 0, or 1
 * when the attributes are malformed.  Host only; no counterpart in the reference's C
 * ABI. */
int disc_ral_conv2d_plan(const char* data_format, const int64_t* strides, int n_strides,
                         const int64_t* dilations, int n_dilations, const char* padding,
                         const int64_t* explicit_paddings, int n_explicit,
                         int weight_is_const, const int64_t in_sizes[4],
                         const int64_t w_sizes[4], int32_t padding_out[4],
                         int32_t metadata_out[17], int64_t result_sizes_out[4]);

/* Parses a serialized custom_attrs blob of `size` bytes (the last operand of every
 * ral_pdll_* call; wire format: R disc/transforms/disc_lower_to_library_call.cc
 * :684-848, reader R ral/context/pdll_util.cc:20-168) and renders it as JSON text
 * into out[0..cap).  Returns the number of bytes the text needs (excluding the NUL),
 * or -1 if the blob is malformed. */
int64_t disc_ral_attr_to_json(const uint8_t* blob, size_t size, char* out, size_t cap);

#ifdef __cplusplus
}
#endif
#endif /* TAO_RAL_API_H_ */
