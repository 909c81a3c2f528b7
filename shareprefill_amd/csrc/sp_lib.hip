// Library identity and the per-thread error string of libshareprefill_hip.
#include <stdarg.h>

#include "sp_common.h"

static thread_local char g_sp_error[512] = "";

void sp_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_sp_error, sizeof(g_sp_error), fmt, ap);
  va_end(ap);
}

extern "C" int sp_version(void) { return 3; }
extern "C" const char* sp_arch(void) { return "gfx950"; }
extern "C" const char* sp_last_error(void) { return g_sp_error; }


// ---- matrix-core rate probe ------------------------------------------------------------------------------
typedef __bf16 diag_bf16x8 __attribute__((ext_vector_type(8)));
typedef float diag_floatx16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(512, 1) void sp_diag_mfma_kernel(float* out, int iters, int random_operands) {
  unsigned h = (threadIdx.x * 2654435761u) ^ (blockIdx.x * 40503u) ^ 0x9e3779b9u;
  auto next = [&]() {
    h ^= h << 13;
    h ^= h >> 17;
    h ^= h << 5;
    // two bf16 values in [0.25, 0.5) with random sign and mantissa, or one constant
    return random_operands ? ((h & 0x807F807Fu) | 0x3E803E80u) : 0x3E803E80u;
  };
  // random_operands 1: one random operand pair per lane, the same for every instruction (the inputs of the
  // multipliers never toggle); 2: four different pairs in rotation, so both operands change with every
  // instruction as they do in a real product
  diag_bf16x8 a[4], b[4];
  for (int u = 0; u < 4; ++u) {
    if (u == 0 || random_operands == 2) {
      a[u] = __builtin_bit_cast(diag_bf16x8, make_uint4(next(), next(), next(), next()));
      b[u] = __builtin_bit_cast(diag_bf16x8, make_uint4(next(), next(), next(), next()));
    } else {
      a[u] = a[0];
      b[u] = b[0];
    }
  }
  diag_floatx16 acc[4];
  for (int i = 0; i < 4; ++i) acc[i] = (diag_floatx16){0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      asm volatile("" : "+v"(a[u]), "+v"(b[u]));  // four live operand pairs, no merging of equal ones
      acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u], b[u], acc[u], 0, 0, 0);
    }
  }
  float s = 0.f;
  for (int i = 0; i < 4; ++i) s += acc[i][0] + acc[i][7];
  if (s == 123.456f) out[threadIdx.x] = s;  // keeps the accumulators alive
}

static int diag_cus() {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 256;
  return prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
}

extern "C" double sp_diag_mfma_flops(int32_t iters) {
  return (double)diag_cus() * 8.0 * 4.0 * (double)iters * 2.0 * 32.0 * 32.0 * 16.0;
}

extern "C" int sp_diag_mfma_bf16(int32_t iters, int32_t random_operands, float* out, sp_stream_t stream) {
  SP_REQUIRE(out && iters > 0, SP_ERR_INVALID_ARGUMENT, "sp_diag_mfma_bf16: bad arguments");
  hipLaunchKernelGGL(sp_diag_mfma_kernel, dim3(diag_cus()), dim3(512), 0, (hipStream_t)stream, out, iters,
                     random_operands);
  SP_LAUNCH_CHECK();
  return SP_OK;
}
