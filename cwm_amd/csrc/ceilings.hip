// What the GPU at hand reaches, measured: the rate at which a kernel can read device memory and the
// rate of the bfloat16 matrix instruction.  The measurement program divides the step's and the prefill's
// rates by these beside the published peaks, so that a fraction says how much is left to the kernels
// rather than to the machine.
//
// The reference measures nothing of the kind; its only throughput line is serve/fgserve.py:330-349.
#include "common.h"

CWM_DEFINE_ERROR_API

#define READ_THREADS 256
#define READ_UNROLL 8  // 16-byte loads a thread has in flight

// Every thread reads 16 bytes at a time, READ_UNROLL of them in flight, a block walking its own contiguous
// share of the buffer (as a product's block walks its tiles of a weight matrix).  The loads' values are
// folded into one word that is stored only if it takes a value that no data gives, so nothing is written.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(READ_THREADS)
read_kernel(const u32x4* __restrict__ src, long n_vec, uint32_t* __restrict__ sink) {
  const long per_block = (n_vec + gridDim.x - 1) / gridDim.x;
  const long begin = (long)blockIdx.x * per_block;
  const long end = begin + per_block < n_vec ? begin + per_block : n_vec;
  uint32_t fold = 0;
  long i = begin + threadIdx.x;
  for (; i + (READ_UNROLL - 1) * READ_THREADS < end; i += READ_UNROLL * READ_THREADS) {
    u32x4 v[READ_UNROLL];
#pragma unroll
    for (int u = 0; u < READ_UNROLL; ++u) v[u] = __builtin_nontemporal_load(src + i + u * READ_THREADS);
#pragma unroll
    for (int u = 0; u < READ_UNROLL; ++u) fold ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < end; i += READ_THREADS) {
    const u32x4 v = __builtin_nontemporal_load(src + i);
    fold ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (fold == 0x9e3779b9u && sink != nullptr) sink[0] = fold;  // the buffer is zeros: never
}

// Reads `bytes` (a multiple of 16) from `src` with `blocks` blocks.
extern "C" int cwm_ceiling_read(const void* src, long bytes, int blocks, void* sink, hipStream_t stream) {
  CWM_REQUIRE(bytes > 0 && bytes % 16 == 0, "ceiling_read: %ld bytes is no positive multiple of 16", bytes);
  CWM_REQUIRE(blocks > 0 && blocks <= (1 << 20), "ceiling_read: %d blocks", blocks);
  CWM_REQUIRE(((uintptr_t)src % 16) == 0, "ceiling_read: the buffer must be 16-byte aligned");
  hipLaunchKernelGGL(read_kernel, dim3((unsigned)blocks), dim3(READ_THREADS), 0, stream, (const u32x4*)src, bytes / 16, (uint32_t*)sink);
  return cwm_launch_status("ceiling_read");
}

#define MFMA_CHAINS 8  // independent accumulators of a wavefront, so that no instruction waits for the one before

typedef float float16v __attribute__((ext_vector_type(16)));

// Every wavefront issues `iters` rounds of MFMA_CHAINS matrix instructions (bfloat16 operands, float32 sums;
// SHAPE 16: 16x16x32, SHAPE 32: 32x32x16, the same number of products each) on operands that stay in
// registers.  The operands are `seed` times small varied numbers: what the instructions cost in power, and
// with that the clock they run at, depends on the data, and operands of zeros would flatter the rate.
// The sums are stored only if they take a value they cannot take.
template <int SHAPE>
__global__ void __launch_bounds__(256)
mfma_kernel(int iters, float seed, float* __restrict__ sink) {
  Frag8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a.h[i] = f32_to_bf16(seed * 0.25f * (float)((int)((threadIdx.x * 7 + i * 3) % 13) - 6));
    b.h[i] = f32_to_bf16(seed * 0.125f * (float)((int)((threadIdx.x * 5 + i * 11) % 17) - 8));
  }
  float total = 0.f;
  if (SHAPE == 16) {
    float4v acc[MFMA_CHAINS];
#pragma unroll
    for (int c = 0; c < MFMA_CHAINS; ++c) acc[c] = float4v{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int c = 0; c < MFMA_CHAINS; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[c], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < MFMA_CHAINS; ++c) total += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
  } else {
    float16v acc[MFMA_CHAINS / 2];
#pragma unroll
    for (int c = 0; c < MFMA_CHAINS / 2; ++c)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[c][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int c = 0; c < MFMA_CHAINS / 2; ++c) {
        acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc[c], 0, 0, 0);
        acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b.v, a.v, acc[c], 0, 0, 0);
      }
    }
#pragma unroll
    for (int c = 0; c < MFMA_CHAINS / 2; ++c) total += acc[c][0] + acc[c][5] + acc[c][10] + acc[c][15];
  }
  if (total == -1.2345e-30f && sink != nullptr) sink[0] = total;
}

// flops of one call: blocks * 4 wavefronts * iters * MFMA_CHAINS instructions of 2 * 16 * 16 * 32 (SHAPE 32: half as
// many chains, two instructions of 2 * 32 * 32 * 16 on each a round: the same number)
extern "C" double cwm_ceiling_mfma_flops(int blocks, int iters) {
  return (double)blocks * 4.0 * (double)iters * MFMA_CHAINS * 2.0 * 16 * 16 * 32;
}

extern "C" int cwm_ceiling_mfma(int blocks, int iters, int shape, float seed, void* sink, hipStream_t stream) {
  CWM_REQUIRE(blocks > 0 && blocks <= (1 << 20) && iters > 0, "ceiling_mfma: %d blocks, %d rounds", blocks, iters);
  CWM_REQUIRE(shape == 16 || shape == 32, "ceiling_mfma: shape %d is neither 16 (16x16x32) nor 32 (32x32x16)", shape);
  if (shape == 16)
    hipLaunchKernelGGL(mfma_kernel<16>, dim3((unsigned)blocks), dim3(256), 0, stream, iters, seed, (float*)sink);
  else
    hipLaunchKernelGGL(mfma_kernel<32>, dim3((unsigned)blocks), dim3(256), 0, stream, iters, seed, (float*)sink);
  return cwm_launch_status("ceiling_mfma");
}
