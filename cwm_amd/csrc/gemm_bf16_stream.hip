// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for at most 64 rows: the matrix product of a
// decode step, bound by reading W once from HBM.  Persistent blocks, one per compute
// unit: each of a block's 16 wavefronts owns a slice of K and keeps its slice of A
// (the matrix-core B operand) in registers for the whole kernel, so A is read once
// per block instead of once per 16 rows of W; the block then walks over 16-row tiles
// of W, every lane streaming 16 contiguous bytes of its row per step with the next
// half tile always in flight, and adds the wavefronts' partial sums through LDS in a
// fixed order.  The sums of a tile are written by rows: 16 adjacent threads write 16
// adjacent columns, one 64-byte request (float32) per row.
//
// When K is too long for the registers, or N gives too few tiles to fill the chip,
// K is split over `k_split` groups of blocks; group g writes float32 partial sums
// C[g][M][N] and the consumer adds them (the residual-add + RMSNorm kernel does, in
// group order).  Every sum's order is fixed by K and k_split alone, so a row's result
// does not depend on how many rows the call has.
//
//   v_mfma_f32_16x16x32_bf16:  C^T[n, m] += W[n, k] * A[m, k]
//     A operand = W tile (lane 16*j + r: row n0 + r, k = 32*s + 8*j .. +7)
//     B operand = A^T    (lane 16*j + r: row r of A, same k)
//     result lane 16*j + r holds C[r][n0 + 4*j + i], i = 0..3
//
// Two shapes of block are built, both of 16 wavefronts: one 16-row tile of A with 12
// steps of K per wavefront in registers (M <= 16, K up to 6144 without a split), and
// four tiles of A with 4 steps of K per wavefront (M <= 64, K up to 2048 per split).
//
// Replaces torch.nn.functional.linear at cwm/fastgen/forward.py:593-606,763,776-782,
// 820 for decode batches.  Needs K % 8 == 0 and 16-byte aligned rows; any N; M <= 64.
#include "common.h"

CWM_DEFINE_ERROR_API

// block shapes: {tiles of A, wavefronts, steps of 32 along K in half a W tile}; a wavefront
// holds 2 * half steps of each of its tiles of A in registers
#ifndef ST1_WAVES
#define ST1_WAVES 16
#endif
#ifndef ST1_HALF
#define ST1_HALF 6
#endif
#ifndef ST4_WAVES
#define ST4_WAVES 16
#endif
#ifndef ST4_HALF
#define ST4_HALF 2
#endif

extern "C" int cwm_gemm_bf16_stream_steps_per_wave(int m) { return m <= 16 ? 2 * ST1_HALF : 2 * ST4_HALF; }
extern "C" int cwm_gemm_bf16_stream_waves(int m) { return m <= 16 ? ST1_WAVES : ST4_WAVES; }

// What the joined q/k/v projection's epilogue needs to rotate queries and keys and to
// put the new keys and values into the paged cache (the work of rope_kv.hip, same
// arithmetic: the sums are rounded to bfloat16 first, then rotated in float32).
struct RopeKv {
  const int* positions;     // [M]
  const int* seq_of_token;  // [M]
  const float* inv_freq;    // [head_dim / 2] or null
  bf16_t* cache;            // [pages][2][n_kv_heads][page_size * head_dim]
  const int* block_table;   // [B][table_width]
  int table_width, page_size, num_pages, n_q_heads, n_kv_heads, head_dim;
};

// ROPE: the output columns are [q heads | k heads | v heads]; q and k are rotated by
// their row's position and k, v are also written to the cache (forward.py:618-632).
//
// TILED: W is the streaming copy of the matrix, [tiles of 16 rows][steps of 32 along K][64 lanes][8 values]:
// lane 16 j + r of a step holds W[16 tile + r][32 step + 8 j ..+8], the operand of one matrix instruction, so
// that a wavefront's load instruction reads 1 KB of consecutive memory, a wavefront's share of a tile is
// consecutive, and so is the tile.  Rows past N and columns past K are zeros there.  Whole cache lines are
// read exactly once, so these loads are non-temporal: they do not displace what the caches hold.  (Measured
// on a kernel that only reads: the 32B shape's gate/up matrix in 78 us this way, 88 to 90 us with either
// the row-major addresses or the ordinary loads, and 100 us with non-temporal loads of the row-major
// addresses, which read every line in two halves.)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename TC, bool ROPE, bool GLU, int MT, int ST_WAVES, int ST_HALF, bool TILED>
__global__ void __launch_bounds__(ST_WAVES * 64)
gemm_stream_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, long ldw, TC* __restrict__ C,
                   long ldc, long split_stride, const void* __restrict__ bias, int bias_dtype, int M, int N, int K,
                   int steps_per_wave, int n_tiles, int k_split, RopeKv rk) {
  __shared__ float red[2][ST_WAVES][MT * 256];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15;
  const int j = lane >> 4;
  const int ks = blockIdx.x % k_split;
  const int tile_first = blockIdx.x / k_split;
  const int tile_stride = gridDim.x / k_split;

  // this wavefront's steps of 32 along K, and its slice of A in registers
  const int s0 = (ks * ST_WAVES + wave) * steps_per_wave;
  const int koff = 32 * s0 + 8 * j;
  Frag8 xf[MT][2 * ST_HALF];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = mt * 16 + r;
    const bf16_t* xrow = A + (size_t)min(row, M - 1) * lda;
#pragma unroll
    for (int i = 0; i < 2 * ST_HALF; ++i) {
      const int k = koff + 32 * i;
      const bool ok = i < steps_per_wave && k + 8 <= K && row < M;
      xf[mt][i].u = ok ? *(const uint4*)(xrow + k) : make_uint4(0, 0, 0, 0);
    }
  }

  const int steps_total = (K + 31) / 32;
  auto load_half = [&](Frag8 (&buf)[ST_HALF], int tile, int half) {
    if (TILED) {
      // ldw: values of one tile (16 rows of all steps)
      const u32x4* wtile = (const u32x4*)(W + (size_t)min(tile, n_tiles - 1) * ldw) + (size_t)s0 * 64 + lane;
#pragma unroll
      for (int i = 0; i < ST_HALF; ++i) {
        const int step = half * ST_HALF + i;
        const bool ok = tile < n_tiles && step < steps_per_wave && s0 + step < steps_total;
        buf[i].w = ok ? __builtin_nontemporal_load(wtile + (size_t)step * 64) : u32x4{0, 0, 0, 0};
      }
      return;
    }
    const bf16_t* wrow = W + (size_t)min(tile * 16 + r, N - 1) * ldw;
#pragma unroll
    for (int i = 0; i < ST_HALF; ++i) {
      const int step = half * ST_HALF + i;
      const int k = koff + 32 * step;
      const bool ok = tile < n_tiles && step < steps_per_wave && k + 8 <= K;
      buf[i].u = ok ? *(const uint4*)(wrow + k) : make_uint4(0, 0, 0, 0);
    }
  };

  Frag8 wa[ST_HALF], wb[ST_HALF];
  int tile = tile_first;
  load_half(wa, tile, 0);
  int parity = 0;
  for (; tile < n_tiles; tile += tile_stride) {
    load_half(wb, tile, 1);
    float4v acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < ST_HALF; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[i].v, xf[mt][i].v, acc[mt], 0, 0, 0);
    load_half(wa, tile + tile_stride, 0);  // the next tile's first half, in flight during the rest of this one
#pragma unroll
    for (int i = 0; i < ST_HALF; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[i].v, xf[mt][ST_HALF + i].v, acc[mt], 0, 0, 0);

    float* mine = red[parity][wave];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(float4v*)(mine + mt * 256 + r * 16 + 4 * j) = acc[mt];  // [row][column]
    __syncthreads();
    if (ROPE) {
      if (threadIdx.x < 128) {
        // a pair of adjacent columns (2i, 2i + 1) of one row
        const int idx = threadIdx.x * 2;
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < ST_WAVES; ++w) {
          s0 += red[parity][w][idx];
          s1 += red[parity][w][idx + 1];
        }
        const int m = idx >> 4;
        const int n = tile * 16 + (idx & 15);
        if (m < M && n + 1 < N) {
          if (bias) {
            s0 += bias_dtype == CWM_BF16 ? bf16_to_f32(((const bf16_t*)bias)[n]) : ((const float*)bias)[n];
            s1 += bias_dtype == CWM_BF16 ? bf16_to_f32(((const bf16_t*)bias)[n + 1]) : ((const float*)bias)[n + 1];
          }
          const bf16_t r0 = f32_to_bf16(s0), r1 = f32_to_bf16(s1);
          const int q_dim = rk.n_q_heads * rk.head_dim;
          const int kv_dim = rk.n_kv_heads * rk.head_dim;
          bf16_t o0 = r0, o1 = r1;
          const bool is_v = n >= q_dim + kv_dim;
          const int pos = rk.positions[m];
          const int d = n % rk.head_dim;
          if (!is_v && rk.inv_freq) {
            float sn, cs;
            sincosf((float)pos * rk.inv_freq[d >> 1], &sn, &cs);
            const float re = bf16_to_f32(r0), im = bf16_to_f32(r1);
            o0 = f32_to_bf16(re * cs - im * sn);
            o1 = f32_to_bf16(im * cs + re * sn);
          }
          bf16_t* crow = (bf16_t*)C + (size_t)m * ldc + n;
          crow[0] = o0;
          crow[1] = o1;
          if (n >= q_dim) {
            const int lp = pos / rk.page_size;
            const int slot = pos - lp * rk.page_size;
            const int page = (lp >= 0 && lp < rk.table_width) ? rk.block_table[(size_t)rk.seq_of_token[m] * rk.table_width + lp] : -1;
            if (page >= 0 && page < rk.num_pages) {
              const size_t plane = (size_t)rk.n_kv_heads * rk.page_size * rk.head_dim;
              bf16_t* base = rk.cache + (size_t)page * 2 * plane;
              if (!is_v) {
                const int head = (n - q_dim) / rk.head_dim;
                bf16_t* dst = base + ((size_t)head * rk.page_size + slot) * rk.head_dim + d;
                dst[0] = o0;
                dst[1] = o1;
              } else {
                const int head = (n - q_dim - kv_dim) / rk.head_dim;
                const int vb = (rk.page_size % 8 == 0) ? 8 : rk.page_size;
                bf16_t* dst = base + plane + (size_t)head * rk.head_dim * rk.page_size +
                              ((size_t)(slot / vb) * rk.head_dim + d) * vb + slot % vb;
                dst[0] = o0;
                dst[vb] = o1;
              }
            }
          }
        }
      }
    } else if (GLU) {
      // rows 16t .. 16t+7 of W are gate rows and 16t+8 .. 16t+15 the up rows of the same 8 columns of
      // the result: thread e finishes row e / 8, column 8t + e % 8 (both sums rounded to bfloat16
      // first, as a product that stored them would have, then silu(gate) * up in float32)
      for (int e = threadIdx.x; e < MT * 128; e += ST_WAVES * 64) {
        const int m = e >> 3;
        const int c = e & 7;
        float gate = 0.f, up = 0.f;
#pragma unroll
        for (int w = 0; w < ST_WAVES; ++w) {
          gate += red[parity][w][m * 16 + c];
          up += red[parity][w][m * 16 + 8 + c];
        }
        const int n = tile * 8 + c;
        if (m < M && 2 * n < N) {
          if (bias) {
            const int nb = tile * 16 + c;
            gate += bias_dtype == CWM_BF16 ? bf16_to_f32(((const bf16_t*)bias)[nb]) : ((const float*)bias)[nb];
            up += bias_dtype == CWM_BF16 ? bf16_to_f32(((const bf16_t*)bias)[nb + 8]) : ((const float*)bias)[nb + 8];
          }
          const float gr = bf16_to_f32(f32_to_bf16(gate)), ur = bf16_to_f32(f32_to_bf16(up));
          Elem<TC>::store(C + (size_t)m * ldc + n, gr / (1.0f + expf(-gr)) * ur);
        }
      }
    } else {
      for (int e = threadIdx.x; e < MT * 256; e += ST_WAVES * 64) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < ST_WAVES; ++w) sum += red[parity][w][e];
        const int m = e >> 4;  // 16 adjacent threads write 16 adjacent columns of a row: one request
        const int n = tile * 16 + (e & 15);
        if (m < M && n < N) {
          if (bias && ks == 0) sum += bias_dtype == CWM_BF16 ? bf16_to_f32(((const bf16_t*)bias)[n]) : ((const float*)bias)[n];
          Elem<TC>::store(C + (size_t)ks * split_stride + (size_t)m * ldc + n, sum);
        }
      }
    }
    // the other buffer is written next; this one again only after the next barrier
    parity ^= 1;
  }
}

extern "C" int cwm_gemm_bf16_stream(const void* A, long lda, const void* W, long ldw, void* C, int c_dtype, long ldc,
                                    long split_stride, const void* bias, int bias_dtype, int M, int N, int K,
                                    int k_split, int n_blocks, const int* rope_positions,
                                    const int* rope_seq_of_token, const float* rope_inv_freq, void* rope_cache,
                                    const int* rope_block_table, int rope_table_width, int rope_page_size,
                                    int rope_num_pages, int rope_n_q_heads, int rope_n_kv_heads, int rope_head_dim,
                                    int glu, int tiled, hipStream_t stream) {
  // tiled != 0: W is the streaming copy (see the kernel; `cwm_gemm_bf16_stream_tiled_values` gives its size) and ldw
  // the values of one of its tiles
  // glu != 0: W holds gate and up rows in alternating groups of 8 and C [M, N / 2] receives
  // silu(gate) * up (cwm/fastgen/forward.py:776-781)
  // rope_positions != null: the columns are [q | k | v] heads; rotate q and k and write k, v to the cache.
  RopeKv rk = {rope_positions, rope_seq_of_token, rope_inv_freq, (bf16_t*)rope_cache, rope_block_table, rope_table_width,
               rope_page_size, rope_num_pages, rope_n_q_heads, rope_n_kv_heads, rope_head_dim};
  const bool rope = rope_positions != nullptr;
  if (rope) {
    CWM_REQUIRE(k_split == 1 && c_dtype == CWM_BF16 && M <= 16, "gemm_bf16_stream: the q/k/v epilogue needs bfloat16 output and no split");
    CWM_REQUIRE(rope_seq_of_token && rope_cache && rope_block_table, "gemm_bf16_stream: cache arguments missing");
    CWM_REQUIRE(rope_head_dim > 0 && rope_head_dim % 2 == 0 && rope_n_q_heads > 0 && rope_n_kv_heads > 0 &&
                    N == (rope_n_q_heads + 2 * rope_n_kv_heads) * rope_head_dim,
                "gemm_bf16_stream: %d columns are not %d + 2 * %d heads of %d", N, rope_n_q_heads, rope_n_kv_heads, rope_head_dim);
    CWM_REQUIRE(rope_page_size > 0 && rope_num_pages > 0 && rope_table_width > 0, "gemm_bf16_stream: bad cache geometry");
  }
  if (glu) {
    CWM_REQUIRE(!rope && k_split == 1 && c_dtype == CWM_BF16 && M <= 16 && N % 16 == 0,
                "gemm_bf16_stream: the gated epilogue needs at most 16 rows, no split, bfloat16 output and N a multiple of 16");
    CWM_REQUIRE(2 * ldc >= N, "gemm_bf16_stream: row stride of the gated result shorter than its rows");
  }
  CWM_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16_stream: bad sizes M=%d N=%d K=%d", M, N, K);
  CWM_REQUIRE(M <= 64, "gemm_bf16_stream: M=%d is more than 64 rows", M);
  const int ST_WAVES = M <= 16 ? ST1_WAVES : ST4_WAVES;
  const int ST_HALF = M <= 16 ? ST1_HALF : ST4_HALF;
  CWM_REQUIRE(K % 8 == 0, "gemm_bf16_stream: K=%d must be a multiple of 8", K);
  CWM_REQUIRE(lda % 8 == 0 && ldw % 8 == 0, "gemm_bf16_stream: row strides must be multiples of 8 elements");
  CWM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_bf16_stream: operands must be 16-byte aligned");
  CWM_REQUIRE(lda >= K && (tiled || ldw >= K) && (glu || ldc >= N), "gemm_bf16_stream: row strides shorter than rows");
  CWM_REQUIRE(!tiled || ldw == (long)((K + 31) / 32) * 512, "gemm_bf16_stream: a tile of the streaming copy has %ld values, not %ld",
              (long)((K + 31) / 32) * 512, ldw);
  CWM_REQUIRE(c_dtype == CWM_F32 || c_dtype == CWM_BF16, "gemm_bf16_stream: unknown output dtype %d", c_dtype);
  CWM_REQUIRE(k_split >= 1, "gemm_bf16_stream: k_split must be at least 1");
  CWM_REQUIRE(k_split == 1 || c_dtype == CWM_F32, "gemm_bf16_stream: partial sums are float32");
  if (M == 0) return 0;
  const int steps = (K + 31) / 32;
  const int steps_per_wave = (steps + k_split * ST_WAVES - 1) / (k_split * ST_WAVES);
  CWM_REQUIRE(steps_per_wave <= 2 * ST_HALF, "gemm_bf16_stream: K=%d needs k_split of at least %d", K,
              (steps + 2 * ST_HALF * ST_WAVES - 1) / (2 * ST_HALF * ST_WAVES));
  const int n_tiles = (N + 15) / 16;
  CWM_REQUIRE(n_blocks >= k_split && n_blocks % k_split == 0, "gemm_bf16_stream: %d blocks do not divide into %d splits",
              n_blocks, k_split);
  CWM_REQUIRE(n_blocks / k_split <= n_tiles, "gemm_bf16_stream: more blocks than tiles");
  dim3 grid(n_blocks);
  dim3 block(ST_WAVES * 64);
#define CWM_LAUNCH_STREAM_AS(TC, ROPE, GLU, MT, WAVES, HALF, TILED)                                                            \
  hipLaunchKernelGGL((gemm_stream_kernel<TC, ROPE, GLU, MT, WAVES, HALF, TILED>), grid, block, 0, stream, (const bf16_t*)A, lda, \
                     (const bf16_t*)W, ldw, (TC*)C, ldc, split_stride, bias, bias_dtype, M, N, K, steps_per_wave,                 \
                     n_tiles, k_split, rk)
#define CWM_LAUNCH_STREAM(TC, ROPE, GLU, MT, WAVES, HALF)           \
  do {                                                              \
    if (tiled)                                                      \
      CWM_LAUNCH_STREAM_AS(TC, ROPE, GLU, MT, WAVES, HALF, true);   \
    else                                                            \
      CWM_LAUNCH_STREAM_AS(TC, ROPE, GLU, MT, WAVES, HALF, false);  \
  } while (0)
  if (rope)
    CWM_LAUNCH_STREAM(bf16_t, true, false, 1, ST1_WAVES, ST1_HALF);
  else if (glu)
    CWM_LAUNCH_STREAM(bf16_t, false, true, 1, ST1_WAVES, ST1_HALF);
  else if (M <= 16 && c_dtype == CWM_F32)
    CWM_LAUNCH_STREAM(float, false, false, 1, ST1_WAVES, ST1_HALF);
  else if (M <= 16)
    CWM_LAUNCH_STREAM(bf16_t, false, false, 1, ST1_WAVES, ST1_HALF);
  else if (c_dtype == CWM_F32)
    CWM_LAUNCH_STREAM(float, false, false, 4, ST4_WAVES, ST4_HALF);
  else
    CWM_LAUNCH_STREAM(bf16_t, false, false, 4, ST4_WAVES, ST4_HALF);
#undef CWM_LAUNCH_STREAM
#undef CWM_LAUNCH_STREAM_AS
  return cwm_launch_status("gemm_bf16_stream");
}

// ---- the streaming copy of a matrix ----------------------------------------------------------------- //
// values of the streaming copy of W [N, K]: tiles of 16 rows by steps of 32 columns, 512 values each
extern "C" long cwm_gemm_bf16_stream_tiled_values(int N, int K) { return (long)((N + 15) / 16) * ((K + 31) / 32) * 512; }

// one thread a lane's 8 values: out[((tile * steps + step) * 64 + 16 j + r) * 8 ..+8] = W[16 tile + r][32 step + 8 j ..+8]
__global__ void __launch_bounds__(256)
stream_copy_kernel(const bf16_t* __restrict__ W, long ldw, bf16_t* __restrict__ out, int N, int K, long n_chunks, int steps) {
  const long c = (long)blockIdx.x * 256 + threadIdx.x;
  if (c >= n_chunks) return;
  const int lane = (int)(c & 63);
  const long ts = c >> 6;
  const int step = (int)(ts % steps);
  const long tile = ts / steps;
  const long row = tile * 16 + (lane & 15);
  const int k = 32 * step + 8 * (lane >> 4);
  Frag8 v;
  v.u = make_uint4(0, 0, 0, 0);
  if (row < N) {
    if (k + 8 <= K && ldw % 8 == 0 && ((uintptr_t)W % 16) == 0) {
      v.u = *(const uint4*)(W + row * ldw + k);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (k + e < K) v.h[e] = W[row * ldw + k + e];
    }
  }
  *(uint4*)(out + c * 8) = v.u;
}

extern "C" int cwm_gemm_bf16_stream_copy(const void* W, long ldw, void* out, int N, int K, hipStream_t stream) {
  CWM_REQUIRE(N > 0 && K > 0 && ldw >= K, "gemm_bf16_stream_copy: bad sizes N=%d K=%d ldw=%ld", N, K, ldw);
  CWM_REQUIRE(((uintptr_t)out % 16) == 0, "gemm_bf16_stream_copy: the copy must be 16-byte aligned");
  const int steps = (K + 31) / 32;
  const long n_chunks = (long)((N + 15) / 16) * steps * 64;
  const long blocks = (n_chunks + 255) / 256;
  CWM_REQUIRE(blocks <= 0x7fffffffL, "gemm_bf16_stream_copy: the matrix is too large");
  hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const bf16_t*)W, ldw, (bf16_t*)out, N, K,
                     n_chunks, steps);
  return cwm_launch_status("gemm_bf16_stream_copy");
}
