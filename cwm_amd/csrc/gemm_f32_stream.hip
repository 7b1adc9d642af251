// C[M, N] = A[M, K] * W[N, K]^T (+ bias) in true float32 for at most 16 rows: the matrix
// product of a decode step on the 32-bit path, bound by reading W once from HBM.  Float32
// operands on v_mfma_f32_16x16x4_f32 (exact products, float32 sums); nothing is rounded
// below float32 before the final store.
//
// The shape of gemm_bf16_stream.hip: persistent blocks, one per compute unit, of 16 wavefronts
// that each own a slice of K and keep their slice of A in registers for the whole kernel; the
// block walks over 16-row tiles of W, every lane streaming 16 contiguous bytes (four values of
// k) of its row per step with the next half tile in flight, and the wavefronts' partial sums
// meet in LDS in a fixed order.  A lane's four values feed four matrix instructions, so lane
// group j supplies k = 16 s + 4 j + e to instruction e: both operands use that pairing, and any
// pairing gives the same sum of products.  A wavefront holds 12 steps (192 values of k) of A,
// a block 3,072; a longer K is split over k_split groups of blocks that write float32 partial
// sums C[g][M][N] for the consumer to add (as the bfloat16 kernel does).
//
//   v_mfma_f32_16x16x4_f32:  C^T[n, m] += W[n, k] * A[m, k]
//     A operand = W tile (lane 16 j + r: row n0 + r), B operand = A^T (lane 16 j + r: row r of A)
//     result lane 16 j + r holds C[r][n0 + 4 j + i], i = 0..3
//
// The order of a row's sums depends on K and k_split alone, not on how many rows the call has;
// it differs from the order of gemm_f32.hip, which takes more rows, by rounding.
//
// Replaces torch.nn.functional.linear at cwm/fastgen/forward.py:593-606,763,776-782,820 for
// decode batches in float32.  Needs K % 4 == 0 and 16-byte aligned rows; any N; M <= 16.
#include "common.h"

CWM_DEFINE_ERROR_API

#define FS_WAVES 16
#define FS_HALF 6  // steps of 16 along K in half a tile of W; a wavefront holds 2 * FS_HALF steps of A

extern "C" int cwm_gemm_f32_stream_steps_per_block() { return FS_WAVES * 2 * FS_HALF; }

template <typename TC>
__global__ void __launch_bounds__(FS_WAVES * 64)
gemm_f32_stream_kernel(const float* __restrict__ A, long lda, const float* __restrict__ W, long ldw, TC* __restrict__ C,
                       long ldc, long split_stride, const void* __restrict__ bias, int bias_dtype, int M, int N, int K,
                       int steps_per_wave, int n_tiles, int k_split) {
  __shared__ float red[2][FS_WAVES][256];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15;
  const int j = lane >> 4;
  const int ks = blockIdx.x % k_split;
  const int tile_first = blockIdx.x / k_split;
  const int tile_stride = gridDim.x / k_split;

  // this wavefront's steps of 16 along K, and its slice of A in registers
  const int s0 = (ks * FS_WAVES + wave) * steps_per_wave;
  const int koff = 16 * s0 + 4 * j;
  float4 xf[2 * FS_HALF];
  {
    const float* xrow = A + (size_t)min(r, M - 1) * lda;
#pragma unroll
    for (int i = 0; i < 2 * FS_HALF; ++i) {
      const int k = koff + 16 * i;
      const bool ok = i < steps_per_wave && k + 4 <= K && r < M;
      xf[i] = ok ? *(const float4*)(xrow + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }

  auto load_half = [&](float4 (&buf)[FS_HALF], int tile, int half) {
    const float* wrow = W + (size_t)min(tile * 16 + r, N - 1) * ldw;
#pragma unroll
    for (int i = 0; i < FS_HALF; ++i) {
      const int step = half * FS_HALF + i;
      const int k = koff + 16 * step;
      const bool ok = tile < n_tiles && step < steps_per_wave && k + 4 <= K;
      buf[i] = ok ? *(const float4*)(wrow + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  auto multiply = [&](const float4 (&buf)[FS_HALF], int half, float4v& acc) {
#pragma unroll
    for (int i = 0; i < FS_HALF; ++i) {
      const float4 w = buf[i], x = xf[half * FS_HALF + i];
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, x.x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, x.y, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, x.z, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, x.w, acc, 0, 0, 0);
    }
  };

  float4 wa[FS_HALF], wb[FS_HALF];
  int tile = tile_first;
  load_half(wa, tile, 0);
  int parity = 0;
  for (; tile < n_tiles; tile += tile_stride) {
    load_half(wb, tile, 1);
    float4v acc = (float4v){0.f, 0.f, 0.f, 0.f};
    multiply(wa, 0, acc);
    load_half(wa, tile + tile_stride, 0);  // the next tile's first half, in flight during the rest of this one
    multiply(wb, 1, acc);

    *(float4v*)(red[parity][wave] + r * 16 + 4 * j) = acc;  // [row][column]
    __syncthreads();
    if (threadIdx.x < 256) {
      const int e = threadIdx.x;
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < FS_WAVES; ++w) sum += red[parity][w][e];
      const int m = e >> 4;  // 16 adjacent threads write 16 adjacent columns of a row: one request
      const int n = tile * 16 + (e & 15);
      if (m < M && n < N) {
        if (bias && ks == 0) sum += bias_dtype == CWM_BF16 ? bf16_to_f32(((const bf16_t*)bias)[n]) : ((const float*)bias)[n];
        Elem<TC>::store(C + (size_t)ks * split_stride + (size_t)m * ldc + n, sum);
      }
    }
    // the other buffer is written next; this one again only after the next barrier
    parity ^= 1;
  }
}

extern "C" int cwm_gemm_f32_stream(const void* A, long lda, const void* W, long ldw, void* C, int c_dtype, long ldc,
                                   long split_stride, const void* bias, int bias_dtype, int M, int N, int K, int k_split,
                                   int n_blocks, hipStream_t stream) {
  CWM_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32_stream: bad sizes M=%d N=%d K=%d", M, N, K);
  CWM_REQUIRE(M <= 16, "gemm_f32_stream: M=%d is more than 16 rows", M);
  CWM_REQUIRE(K % 4 == 0, "gemm_f32_stream: K=%d must be a multiple of 4", K);
  CWM_REQUIRE(lda % 4 == 0 && ldw % 4 == 0, "gemm_f32_stream: row strides must be multiples of 4 elements");
  CWM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_f32_stream: operands must be 16-byte aligned");
  CWM_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32_stream: row strides shorter than rows");
  CWM_REQUIRE(c_dtype == CWM_F32 || c_dtype == CWM_BF16, "gemm_f32_stream: unknown output dtype %d", c_dtype);
  CWM_REQUIRE(k_split >= 1, "gemm_f32_stream: k_split must be at least 1");
  CWM_REQUIRE(k_split == 1 || c_dtype == CWM_F32, "gemm_f32_stream: partial sums are float32");
  if (M == 0) return 0;
  const int steps = (K + 15) / 16;
  const int steps_per_wave = (steps + k_split * FS_WAVES - 1) / (k_split * FS_WAVES);
  CWM_REQUIRE(steps_per_wave <= 2 * FS_HALF, "gemm_f32_stream: K=%d needs k_split of at least %d", K,
              (steps + 2 * FS_HALF * FS_WAVES - 1) / (2 * FS_HALF * FS_WAVES));
  const int n_tiles = (N + 15) / 16;
  CWM_REQUIRE(n_blocks >= k_split && n_blocks % k_split == 0, "gemm_f32_stream: %d blocks do not divide into %d splits",
              n_blocks, k_split);
  CWM_REQUIRE(n_blocks / k_split <= n_tiles, "gemm_f32_stream: more blocks than tiles");
  dim3 grid(n_blocks);
  dim3 block(FS_WAVES * 64);
  if (c_dtype == CWM_F32)
    hipLaunchKernelGGL(gemm_f32_stream_kernel<float>, grid, block, 0, stream, (const float*)A, lda, (const float*)W, ldw,
                       (float*)C, ldc, split_stride, bias, bias_dtype, M, N, K, steps_per_wave, n_tiles, k_split);
  else
    hipLaunchKernelGGL(gemm_f32_stream_kernel<bf16_t>, grid, block, 0, stream, (const float*)A, lda, (const float*)W, ldw,
                       (bf16_t*)C, ldc, split_stride, bias, bias_dtype, M, N, K, steps_per_wave, n_tiles, k_split);
  return cwm_launch_status("gemm_f32_stream");
}
