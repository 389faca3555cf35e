/* A hand-written stand-in for what the DISC compiler emits for one quantized linear
 * layer: a `main` that receives {execution context, tao_ral_call_impl} and drives the
 * runtime purely through mangled entry names and void** argument slots
 * (argument packing as in tao_compiler/mlir/disc/transforms/disc_to_llvm.cc:74-330).
 *
 *   x   = ral_recv_input(0)                      f32 [M, K]   (device)
 *   w, b, s_w, s_x, s_o, zero = ral_const(...)   from the program's constant store
 *   xq  = quantize(x, s_x)                       i8  [M, K]
 *   yq  = ral_pdll_qgemm(xq, w, b, ...)          i8  [M, N]   (callee-allocated)
 *   y   = dequantize(yq, s_o)                    f32 [M, N]
 *   ral_send_output(0, y)
 *
 * Test fixture only; compiled with gcc by tests/test_gpu_program.py. */
#include <stdint.h>
#include <string.h>
#include <time.h>

typedef void (*ral_call_t)(void* exec, void* name, void** args);

typedef struct { void* base; void* data; int64_t offset; } MemRef0;
typedef struct { void* base; void* data; int64_t offset; int64_t sizes[1]; int64_t strides[1]; } MemRef1;
typedef struct { void* base; void* data; int64_t offset; int64_t sizes[2]; int64_t strides[2]; } MemRef2;

/* the custom_attrs blob of the ral_pdll_qgemm call; filled in by the test harness */
extern const unsigned char kQgemmAttrs[];

static int push0(void** a, int n, MemRef0* m) { a[n++] = &m->base; a[n++] = &m->data; a[n++] = &m->offset; return n; }
static int push1(void** a, int n, MemRef1* m) { n = push0(a, n, (MemRef0*)m); a[n++] = &m->sizes[0]; a[n++] = &m->strides[0]; return n; }
static int push2(void** a, int n, MemRef2* m) {
  n = push0(a, n, (MemRef0*)m);
  a[n++] = &m->sizes[0]; a[n++] = &m->sizes[1]; a[n++] = &m->strides[0]; a[n++] = &m->strides[1];
  return n;
}

static void* const_call(ral_call_t call, void* exec, const char* entry, const char* name, int32_t index,
                        void* result) {
  void* stream = 0;
  const char* unique_name = name;
  void* args[5] = {&exec, &stream, &unique_name, &index, result};
  call(exec, (void*)entry, args);
  return result;
}

static void* gpu_alloc(ral_call_t call, void* exec, int64_t bytes) {
  void* ptr = 0;
  void* args[3] = {&exec, &bytes, &ptr};
  call(exec, (void*)"alloc___gpu___pvoid_i64___pvoid", args);
  return ptr;
}

static void gpu_dealloc(ral_call_t call, void* exec, void* ptr) {
  void* args[2] = {&exec, &ptr};
  call(exec, (void*)"dealloc___gpu___pvoid_pvoid___void", args);
}

/* input -> constants -> quantize -> ral_pdll_qgemm: the part both programs share */
typedef struct {
  void* exec; ral_call_t call; void* stream;
  MemRef2 x, yq; MemRef0 so, zero;
  int64_t M, N;
} Front;

static void run_front(void** ctx_struct, Front* f) {
  void* exec = ctx_struct[0];
  ral_call_t call = (ral_call_t)ctx_struct[1];
  void* stream = 0;   /* stream index 0 */

  /* ---- input */
  MemRef2 x;
  { int64_t idx = 0; void* args[3] = {&exec, &idx, &x};
    call(exec, (void*)"ral_recv_input___cpu___pvoid_i64___m2df32", args); }
  const int64_t M = x.sizes[0], K = x.sizes[1];

  /* ---- constants */
  MemRef2 w; MemRef1 bias, sw; MemRef0 sx, so, zero;
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m2di8", "w0_i8_768x768", 0, &w);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m1df32", "b0_f32_768", 1, &bias);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m1df32", "sw0_f32_768", 2, &sw);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m0df32", "sx0_f32_", 3, &sx);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m0df32", "so0_f32_", 4, &so);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m0di32", "z0_i32_", 5, &zero);
  const int64_t N = w.sizes[0];

  /* ---- xq = quantize(x) */
  MemRef2 xq = {0};
  xq.base = xq.data = gpu_alloc(call, exec, M * K);
  xq.sizes[0] = M; xq.sizes[1] = K; xq.strides[0] = K; xq.strides[1] = 1;
  { void* args[32]; int n = 0;
    int64_t axis = -1, qmin = -128, qmax = 127, round_mode = 1;
    args[n++] = &exec; args[n++] = &stream;
    n = push2(args, n, &x); n = push0(args, n, &sx); n = push0(args, n, &zero); n = push2(args, n, &xq);
    args[n++] = &axis; args[n++] = &qmin; args[n++] = &qmax; args[n++] = &round_mode;
    call(exec, (void*)"ral_quantize___gpu___pvoid_pvoid_m2df32_m0df32_m0di32_m2di8_i64_i64_i64_i64___void", args); }

  /* ---- yq = ral_pdll_qgemm(xq, w[N,K], bias f32, ...), zero points are host values */
  MemRef2 yq;
  { int32_t zx = 0, zo = 0; int32_t zw_data[768]; memset(zw_data, 0, sizeof(zw_data));
    MemRef0 zx_m = {&zx, &zx, 0}, zo_m = {&zo, &zo, 0};
    MemRef1 zw_m = {zw_data, zw_data, 0, {N}, {1}};
    const void* attrs = kQgemmAttrs;
    void* args[64]; int n = 0;
    args[n++] = &exec; args[n++] = &stream;
    n = push2(args, n, &xq); n = push2(args, n, &w); n = push1(args, n, &bias);
    n = push0(args, n, &sx); n = push0(args, n, &zx_m);
    n = push1(args, n, &sw); n = push1(args, n, &zw_m);
    n = push0(args, n, &so); n = push0(args, n, &zo_m);
    args[n++] = &attrs; args[n++] = &yq;
    call(exec, (void*)"ral_pdll_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m1df32_m0df32_m0di32_m1df32_m1di32_m0df32_m0di32_pvoid___m2di8", args); }
  gpu_dealloc(call, exec, xq.data);

  f->exec = exec; f->call = call; f->stream = stream;
  f->x = x; f->yq = yq; f->so = so; f->zero = zero; f->M = M; f->N = N;
}

static void send_outputs(Front* f, MemRef2* y) {
  void* exec = f->exec; ral_call_t call = f->call;
  /* ---- output 0 = y; output 1 = x (an input forwarded unchanged) */
  { int64_t idx = 0; void* args[16]; int n = 0; args[n++] = &exec; args[n++] = &idx; n = push2(args, n, y);
    call(exec, (void*)"ral_send_output___cpu___pvoid_i64_m2df32___void", args); }
  { int64_t idx = 1; void* args[16]; int n = 0; args[n++] = &exec; args[n++] = &idx; n = push2(args, n, &f->x);
    call(exec, (void*)"ral_send_output___cpu___pvoid_i64_m2df32___void", args); }
}

void disc_program_main(void** ctx_struct) {
  Front f; run_front(ctx_struct, &f);
  void* exec = f.exec; ral_call_t call = f.call; void* stream = f.stream;
  MemRef2 yq = f.yq; MemRef0 so = f.so, zero = f.zero; const int64_t M = f.M, N = f.N;
  /* ---- y = dequantize(yq) */
  MemRef2 y = {0};
  y.base = y.data = gpu_alloc(call, exec, M * N * 4);
  y.sizes[0] = M; y.sizes[1] = N; y.strides[0] = N; y.strides[1] = 1;
  { void* args[32]; int n = 0; int64_t axis = -1;
    args[n++] = &exec; args[n++] = &stream;
    n = push2(args, n, &yq); n = push0(args, n, &so); n = push0(args, n, &zero); n = push2(args, n, &y);
    args[n++] = &axis;
    call(exec, (void*)"ral_dequantize___gpu___pvoid_pvoid_m2di8_m0df32_m0di32_m2df32_i64___void", args); }
  gpu_dealloc(call, exec, yq.data);

  send_outputs(&f, &y);
}

/* The same program with the dequantize replaced by a fused elementwise kernel that the
 * compiler would have generated and embedded as a code object:
 * y = relu(dequantize(yq)) + x, launched through ral_kernel_launch (N must equal K). */
static const void* g_code_objects[8] = {0};
static int64_t g_num_code_objects = 0;
void disc_program_set_code_object(const void* blob) { g_code_objects[0] = blob; g_num_code_objects = 1; }
/* Several images for one kernel, as a build for more than one processor carries them. */
void disc_program_set_code_objects(const void** blobs, int64_t n) {
  g_num_code_objects = n < 8 ? n : 8;
  for (int64_t i = 0; i < g_num_code_objects; ++i) g_code_objects[i] = blobs[i];
}

void disc_program_main_fused(void** ctx_struct) {
  Front f; run_front(ctx_struct, &f);
  void* exec = f.exec; ral_call_t call = f.call; void* stream = f.stream;
  const int64_t M = f.M, N = f.N;
  MemRef2 y = {0};
  y.base = y.data = gpu_alloc(call, exec, M * N * 4);
  y.sizes[0] = M; y.sizes[1] = N; y.strides[0] = N; y.strides[1] = 1;
  { void* blobs[8]; for (int i = 0; i < 8; ++i) blobs[i] = (void*)g_code_objects[i];
    void** blobs_p = blobs; int64_t num_blobs = g_num_code_objects;
    const char* name = "fused_dequant_relu_residual";
    int64_t total = M * N;
    int64_t gx = (total + 255) / 256, gy = 1, gz = 1, bx = 256, by = 1, bz = 1;
    int32_t smem = 0, num_args = 5;
    void* params[5] = {&f.yq.data, &f.so.data, &f.x.data, &y.data, &total};
    void** params_p = params;
    void* args[14] = {&exec, &blobs_p, &num_blobs, &name, &gx, &gy, &gz, &bx, &by, &bz, &smem,
                      &stream, &num_args, &params_p};
    call(exec, (void*)"ral_kernel_launch___gpu___pvoid_ppvoid_i64_pvoid_i64_i64_i64_i64_i64_i64_i32_pvoid_i32_ppvoid___void", args); }
  gpu_dealloc(call, exec, f.yq.data);
  send_outputs(&f, &y);
}

/* Host cost of the dispatch path: `n` back-to-back ral_pdll_qgemm calls on M rows of
 * uninitialised int8 data (each call allocates its result, which is freed at once), one
 * stream synchronisation at the end.  Returns microseconds per call. */
double disc_program_qgemm_loop(void** ctx_struct, int64_t M, int n) {
  void* exec = ctx_struct[0];
  ral_call_t call = (ral_call_t)ctx_struct[1];
  void* stream = 0;
  MemRef2 w; MemRef1 bias, sw; MemRef0 sx, so;
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m2di8", "w0_i8_768x768", 0, &w);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m1df32", "b0_f32_768", 1, &bias);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m1df32", "sw0_f32_768", 2, &sw);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m0df32", "sx0_f32_", 3, &sx);
  const_call(call, exec, "ral_const___gpu___pvoid_pvoid_pvoid_i32___m0df32", "so0_f32_", 4, &so);
  const int64_t N = w.sizes[0], K = w.sizes[1];
  MemRef2 xq = {0};
  xq.base = xq.data = gpu_alloc(call, exec, M * K);
  xq.sizes[0] = M; xq.sizes[1] = K; xq.strides[0] = K; xq.strides[1] = 1;
  int32_t zx = 0, zo = 0; int32_t zw_data[768]; memset(zw_data, 0, sizeof(zw_data));
  MemRef0 zx_m = {&zx, &zx, 0}, zo_m = {&zo, &zo, 0};
  MemRef1 zw_m = {zw_data, zw_data, 0, {N}, {1}};
  const void* attrs = kQgemmAttrs;
  struct timespec t0, t1;
  clock_gettime(CLOCK_MONOTONIC, &t0);
  for (int it = 0; it < n; ++it) {
    MemRef2 yq;
    void* args[64]; int k = 0;
    args[k++] = &exec; args[k++] = &stream;
    k = push2(args, k, &xq); k = push2(args, k, &w); k = push1(args, k, &bias);
    k = push0(args, k, &sx); k = push0(args, k, &zx_m);
    k = push1(args, k, &sw); k = push1(args, k, &zw_m);
    k = push0(args, k, &so); k = push0(args, k, &zo_m);
    args[k++] = &attrs; args[k++] = &yq;
    call(exec, (void*)"ral_pdll_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m1df32_m0df32_m0di32_m1df32_m1di32_m0df32_m0di32_pvoid___m2di8", args);
    gpu_dealloc(call, exec, yq.data);
  }
  { void* args[2] = {&exec, &stream};
    call(exec, (void*)"sync_on_stream___gpu___pvoid_pvoid___void", args); }
  clock_gettime(CLOCK_MONOTONIC, &t1);
  gpu_dealloc(call, exec, xq.data);
  return ((t1.tv_sec - t0.tv_sec) * 1e6 + (t1.tv_nsec - t0.tv_nsec) * 1e-3) / n;
}
