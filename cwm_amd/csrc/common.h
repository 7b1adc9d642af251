// Shared helpers of the gfx950 kernels: element types, bfloat16 conversion,
// wavefront reductions (64 lanes) and the error channel of the C entry points.
//
// Every entry point is `extern "C" int name(..., hipStream_t stream)`, returns 0
// on success and a non-zero code after storing a message that the caller fetches
// with `cwm_error_message()`.  Entry points check sizes before they launch and
// refuse what a kernel does not cover; they never fall back to another result.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef uint16_t bf16_t;

enum CwmDType : int { CWM_F32 = 0, CWM_BF16 = 1 };

#define CWM_WAVE 64

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest, ties to even; NaN stays NaN (gfx950 converts in hardware: v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const __bf16 h = (__bf16)f;
  return __builtin_bit_cast(bf16_t, h);
}

// two values into one 32-bit word, `lo` in the low half
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  typedef __bf16 cwm_bf16x2 __attribute__((ext_vector_type(2)));
  typedef float cwm_f32x2 __attribute__((ext_vector_type(2)));
  const cwm_f32x2 v = {lo, hi};
  const cwm_bf16x2 h = __builtin_convertvector(v, cwm_bf16x2);
  return __builtin_bit_cast(uint32_t, h);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = CWM_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, CWM_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = CWM_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, CWM_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads in a fixed order (wave shuffles, then the
// wave partials in index order); every thread gets the result.  `scratch` holds at
// least 16 floats of LDS.  Safe to call repeatedly.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const int wave = threadIdx.x / CWM_WAVE;
  const int nwaves = (blockDim.x + CWM_WAVE - 1) / CWM_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const int wave = threadIdx.x / CWM_WAVE;
  const int nwaves = (blockDim.x + CWM_WAVE - 1) / CWM_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// Operands and results of the matrix-core instructions: eight bfloat16 values of one lane
// (16 bytes, also as one load) and the four float32 sums of one lane.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

union Frag8 {
  uint4 u;
  bf16x8 v;
  uint16_t h[8];
  uint32_t __attribute__((ext_vector_type(4))) w;  // the same 16 bytes as a vector the non-temporal load builtin takes
};

// Direct load from global memory into LDS (global_load_lds_dwordx4): every lane's 16 bytes at
// base + offset go to LDS byte address lds + 16 * lane (base and lds are uniform over the
// wavefront).  The load counts in vmcnt like any other; the compiler does not know of it, so
// whoever issues it also writes the waits (s_waitcnt vmcnt) before the LDS is read.
__device__ __forceinline__ void dma16(const bf16_t* base, uint32_t offset, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds), "v"(offset), "s"(base) : "memory", "m0");
}

// The same past the caches (non-temporal): for data that is read once, in whole cache lines per instruction.
__device__ __forceinline__ void dma16_once(const bf16_t* base, uint32_t offset, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" : : "s"(lds), "v"(offset), "s"(base) : "memory", "m0");
}

// ---- host side: error channel ------------------------------------------------ //
static thread_local char cwm_error_buffer[512] = {0};

static inline int cwm_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(cwm_error_buffer, sizeof(cwm_error_buffer), fmt, ap);
  va_end(ap);
  return 1;
}

static inline int cwm_launch_status(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return cwm_fail("%s: launch failed: %s", what, hipGetErrorString(err));
  return 0;
}

#define CWM_DEFINE_ERROR_API \
  extern "C" const char* cwm_error_message() { return cwm_error_buffer; }

#define CWM_REQUIRE(cond, ...) \
  do {                         \
    if (!(cond)) return cwm_fail(__VA_ARGS__); \
  } while (0)
