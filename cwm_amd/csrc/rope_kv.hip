// Rotary position encoding of queries and keys fused with the write of the new
// keys and values into the paged cache.
//
// Rotation (cwm/fastgen/kernels/rope.py:55-90): for pair i of a head,
//   a = float(pos) * inv_freq[i];  (x[2i], x[2i+1]) <- (x[2i] cos a - x[2i+1] sin a,
//                                                      x[2i+1] cos a + x[2i] sin a)
// in float32, the same for every head, applied to queries and keys and not to
// values, before the cache write (cwm/fastgen/forward.py:618-632).
//
// Cache layout of one layer: [num_pages][2][n_kv_heads][page_size * head_dim];
// plane 0 holds keys as [slot][dim]; plane 1 holds values in blocks of VB keys as
// [slot / VB][dim][slot % VB], VB = 8 if the page size is a multiple of 8 and the
// whole page otherwise, so that a matrix-core operand of the attention kernel (one
// dimension, 8 consecutive keys) is 16 contiguous bytes.  The row of a token is
// block_table[seq][pos / page_size], slot pos % page_size
// (cwm/fastgen/kernels/paged_memcpy.py:56-87 computes the same address).
#include "common.h"

CWM_DEFINE_ERROR_API

// bfloat16, head sizes of a multiple of 8: a thread takes four adjacent pairs (16 bytes) of a
// head, computes their four rotations once and applies them to that piece of every head of
// the token; keys go to the cache in the same 16-byte pieces.  Values: as in the kernel below.
// PARTIALS: q, k and v are not read but made here, from the float32 partial sums
// partials[p][t][q heads | k heads | v heads] of the joined projection whose K was split: added in
// order and rounded to bfloat16, as the kernel that adds partial sums would have stored them.
template <bool PARTIALS>
__global__ void rope_kv_write_bf16x8_kernel(bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ k, long k_stride,
                                            bf16_t* __restrict__ v, long v_stride, const int* __restrict__ positions,
                                            const int* __restrict__ seq_of_token, const float* __restrict__ inv_freq,
                                            bf16_t* __restrict__ cache, const int* __restrict__ block_table,
                                            int table_width, int page_size, int num_pages, int n_q_heads, int n_kv_heads,
                                            int head_dim, const float* __restrict__ partials, int n_partials,
                                            long partial_stride) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int pieces = head_dim / 8;
  const int piece = threadIdx.x;  // < pieces
  const int n_heads = n_q_heads + (k ? n_kv_heads : 0);
  bf16_t* kdst = nullptr;
  bf16_t* vdst = nullptr;
  int slot = 0;
  if (cache) {
    const int seq = seq_of_token[t];
    const int lp = pos / page_size;
    slot = pos - lp * page_size;
    const int page = (lp >= 0 && lp < table_width) ? block_table[(size_t)seq * table_width + lp] : -1;
    if (page >= 0 && page < num_pages) {
      const size_t plane = (size_t)n_kv_heads * page_size * head_dim;
      kdst = cache + (size_t)page * 2 * plane;
      vdst = kdst + plane;
    }
  }
  if (piece < pieces) {
    float c[4], s[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      c[e] = 1.f;
      s[e] = 0.f;
      if (inv_freq) sincosf((float)pos * inv_freq[4 * piece + e], &s[e], &c[e]);
    }
    // the blocks of a token (gridDim.y of them) take the heads in turn
    for (int hh = blockIdx.y * blockDim.y + threadIdx.y; hh < n_heads; hh += gridDim.y * blockDim.y) {
      const bool is_key = hh >= n_q_heads;
      const int head = is_key ? hh - n_q_heads : hh;
      bf16_t* row = (is_key ? k + (size_t)t * k_stride : q + (size_t)t * q_stride) + (size_t)head * head_dim + 8 * piece;
      uint32_t w[4];
      if constexpr (PARTIALS) {
        const float* src = partials + (size_t)t * (n_q_heads + 2 * n_kv_heads) * head_dim + (size_t)hh * head_dim + 8 * piece;
        float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
        for (int p = 0; p < n_partials; ++p) {
          const float4 a = *(const float4*)(src + (size_t)p * partial_stride);
          const float4 b = *(const float4*)(src + (size_t)p * partial_stride + 4);
          lo.x += a.x, lo.y += a.y, lo.z += a.z, lo.w += a.w;
          hi.x += b.x, hi.y += b.y, hi.z += b.z, hi.w += b.w;
        }
        w[0] = pack2_bf16(lo.x, lo.y), w[1] = pack2_bf16(lo.z, lo.w), w[2] = pack2_bf16(hi.x, hi.y), w[3] = pack2_bf16(hi.z, hi.w);
      } else {
        const uint4 in = *(const uint4*)row;
        w[0] = in.x, w[1] = in.y, w[2] = in.z, w[3] = in.w;
      }
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float re = bf16_to_f32((bf16_t)(w[e] & 0xffffu));
        const float im = bf16_to_f32((bf16_t)(w[e] >> 16));
        o[e] = (uint32_t)f32_to_bf16(re * c[e] - im * s[e]) | ((uint32_t)f32_to_bf16(im * c[e] + re * s[e]) << 16);
      }
      const uint4 out = make_uint4(o[0], o[1], o[2], o[3]);
      if (inv_freq || PARTIALS) *(uint4*)row = out;
      if (is_key && kdst) *(uint4*)(kdst + ((size_t)head * page_size + slot) * head_dim + 8 * piece) = out;
    }
  }
  if ((vdst || PARTIALS) && v) {
    const int v_block = (page_size % 8 == 0) ? 8 : page_size;
    const int tid = (blockIdx.y * blockDim.y + threadIdx.y) * blockDim.x + threadIdx.x;
    const int nthreads = gridDim.y * blockDim.x * blockDim.y;
    const int total = n_kv_heads * head_dim;
    bf16_t* vrow = v + (size_t)t * v_stride;
    for (int e = tid; e < total; e += nthreads) {
      const int head = e / head_dim;
      const int d = e - head * head_dim;
      bf16_t value;
      if constexpr (PARTIALS) {
        const float* src = partials + ((size_t)t * (n_q_heads + 2 * n_kv_heads) + n_q_heads + n_kv_heads) * head_dim + e;
        float sum = 0.f;
        for (int p = 0; p < n_partials; ++p) sum += src[(size_t)p * partial_stride];
        value = f32_to_bf16(sum);
        vrow[e] = value;
      } else {
        value = vrow[e];
      }
      if (vdst) vdst[(size_t)head * head_dim * page_size + ((size_t)(slot / v_block) * head_dim + d) * v_block + slot % v_block] = value;
    }
  }
}

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ q, long q_stride, T* __restrict__ k, long k_stride,
                                     const T* __restrict__ v, long v_stride,
                                     const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                     const float* __restrict__ inv_freq, T* __restrict__ cache,
                                     const int* __restrict__ block_table, int table_width, int page_size,
                                     int num_pages, int n_q_heads, int n_kv_heads, int head_dim) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = head_dim / 2;
  const int i = threadIdx.x;  // pair index, < half
  const int n_heads = n_q_heads + (k ? n_kv_heads : 0);

  // where this token's key and value go
  T* kdst = nullptr;
  T* vdst = nullptr;
  int slot = 0;
  if (cache) {
    const int seq = seq_of_token[t];
    const int lp = pos / page_size;
    slot = pos - lp * page_size;
    const int page = (lp >= 0 && lp < table_width) ? block_table[(size_t)seq * table_width + lp] : -1;
    if (page >= 0 && page < num_pages) {
      const size_t plane = (size_t)n_kv_heads * page_size * head_dim;
      kdst = cache + (size_t)page * 2 * plane;
      vdst = kdst + plane;
    }
  }

  if (i < half) {
    float c = 1.f, s = 0.f;
    if (inv_freq) {
      const float a = (float)pos * inv_freq[i];
      sincosf(a, &s, &c);
    }
    for (int hh = threadIdx.y; hh < n_heads; hh += blockDim.y) {
      T* row;
      const bool is_key = hh >= n_q_heads;
      const int head = is_key ? hh - n_q_heads : hh;
      if (is_key)
        row = k + (size_t)t * k_stride + (size_t)head * head_dim;
      else
        row = q + (size_t)t * q_stride + (size_t)head * head_dim;
      const float re = Elem<T>::load(row + 2 * i);
      const float im = Elem<T>::load(row + 2 * i + 1);
      const float ore = re * c - im * s;
      const float oim = im * c + re * s;
      if (inv_freq) {
        Elem<T>::store(row + 2 * i, ore);
        Elem<T>::store(row + 2 * i + 1, oim);
      }
      if (is_key && kdst) {
        T* dst = kdst + ((size_t)head * page_size + slot) * head_dim;
        Elem<T>::store(dst + 2 * i, ore);
        Elem<T>::store(dst + 2 * i + 1, oim);
      }
    }
  }

  if (vdst && v) {
    const int v_block = (page_size % 8 == 0) ? 8 : page_size;
    const int tid = threadIdx.y * blockDim.x + threadIdx.x;
    const int nthreads = blockDim.x * blockDim.y;
    const int total = n_kv_heads * head_dim;
    const T* vrow = v + (size_t)t * v_stride;
    for (int e = tid; e < total; e += nthreads) {
      const int head = e / head_dim;
      const int d = e - head * head_dim;
      vdst[(size_t)head * head_dim * page_size + ((size_t)(slot / v_block) * head_dim + d) * v_block + slot % v_block] = vrow[e];
    }
  }
}

extern "C" int cwm_rope_kv_write(void* q, long q_stride, void* k, long k_stride, const void* v, long v_stride,
                                 int dtype, const int* positions, const int* seq_of_token, const float* inv_freq,
                                 void* cache, const int* block_table, int table_width, int page_size,
                                 int num_pages, int n_tokens, int n_q_heads, int n_kv_heads, int head_dim,
                                 hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0, "rope_kv_write: negative token count");
  CWM_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= 1024,
              "rope_kv_write: head_dim %d must be even and at most 1024", head_dim);
  CWM_REQUIRE(n_q_heads >= 0 && n_kv_heads >= 0 && n_q_heads + n_kv_heads > 0, "rope_kv_write: no heads");
  CWM_REQUIRE(q || n_q_heads == 0, "rope_kv_write: queries missing");
  if (cache) {
    CWM_REQUIRE(k && v && block_table && seq_of_token, "rope_kv_write: a cache write needs k, v and a block table");
    CWM_REQUIRE(page_size > 0 && num_pages > 0 && table_width > 0, "rope_kv_write: bad cache geometry");
  }
  if (n_tokens == 0) return 0;
  const int half = head_dim / 2;
  int bx = 1;
  while (bx < half) bx <<= 1;  // threads beyond `half` idle in the rotation
  int by = 256 / bx;
  if (by < 1) by = 1;
  const int heads = n_q_heads + n_kv_heads;
  if (by > heads) by = heads;
  dim3 block(bx, by);
  const bool rows16 = q_stride % 8 == 0 && k_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 &&
                      ((uintptr_t)cache % 16) == 0;
  if (dtype == CWM_BF16 && head_dim % 8 == 0 && head_dim <= 2048 && rows16) {
    int px = 1;
    while (px < head_dim / 8) px <<= 1;
    int py = 256 / px;
    if (py < 1) py = 1;
    if (py > heads) py = heads;
    // few tokens: several blocks a token, so that a decode step's rows are not left to as many blocks
    const int gy = n_tokens >= 1024 ? 1 : (heads + py - 1) / py;
    hipLaunchKernelGGL(rope_kv_write_bf16x8_kernel<false>, dim3(n_tokens, gy), dim3(px, py), 0, stream, (bf16_t*)q, q_stride,
                       (bf16_t*)k, k_stride, (bf16_t*)v, v_stride, positions, seq_of_token, inv_freq, (bf16_t*)cache,
                       block_table, table_width, page_size, num_pages, n_q_heads, n_kv_heads, head_dim, (const float*)nullptr, 0,
                       0L);
  } else if (dtype == CWM_F32)
    hipLaunchKernelGGL(rope_kv_write_kernel<float>, dim3(n_tokens), block, 0, stream, (float*)q, q_stride,
                       (float*)k, k_stride, (const float*)v, v_stride, positions, seq_of_token, inv_freq,
                       (float*)cache, block_table, table_width, page_size, num_pages, n_q_heads, n_kv_heads,
                       head_dim);
  else if (dtype == CWM_BF16)
    hipLaunchKernelGGL(rope_kv_write_kernel<bf16_t>, dim3(n_tokens), block, 0, stream, (bf16_t*)q, q_stride,
                       (bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, positions, seq_of_token, inv_freq,
                       (bf16_t*)cache, block_table, table_width, page_size, num_pages, n_q_heads, n_kv_heads,
                       head_dim);
  else
    return cwm_fail("rope_kv_write: unknown dtype %d", dtype);
  return cwm_launch_status("rope_kv_write");
}

// The same from the float32 partial sums [n_partials][n_tokens][(Hq + 2 Hkv) * head_dim] of the joined
// q/k/v projection (partial_stride elements apart): `qkv` [n_tokens][qkv_stride] receives the sums
// in bfloat16, q and k rotated, and the cache the rotated keys and the values.
extern "C" int cwm_rope_kv_write_partials(void* qkv, long qkv_stride, const float* partials, int n_partials,
                                          long partial_stride, const int* positions, const int* seq_of_token,
                                          const float* inv_freq, void* cache, const int* block_table, int table_width,
                                          int page_size, int num_pages, int n_tokens, int n_q_heads, int n_kv_heads,
                                          int head_dim, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && n_partials >= 1, "rope_kv_write_partials: bad sizes");
  CWM_REQUIRE(head_dim > 0 && head_dim % 8 == 0 && head_dim <= 2048, "rope_kv_write_partials: head_dim %d must be a multiple of 8", head_dim);
  CWM_REQUIRE(n_q_heads > 0 && n_kv_heads > 0, "rope_kv_write_partials: no heads");
  const long width = (long)(n_q_heads + 2 * n_kv_heads) * head_dim;
  CWM_REQUIRE(qkv && partials && positions, "rope_kv_write_partials: arguments missing");
  CWM_REQUIRE(qkv_stride >= width && qkv_stride % 8 == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)partials % 16) == 0 &&
                  partial_stride % 4 == 0 && partial_stride >= (long)n_tokens * width,
              "rope_kv_write_partials: rows must be 16-byte aligned and the partial sums dense");
  if (cache) {
    CWM_REQUIRE(block_table && seq_of_token, "rope_kv_write_partials: a cache write needs a block table");
    CWM_REQUIRE(page_size > 0 && num_pages > 0 && table_width > 0 && ((uintptr_t)cache % 16) == 0, "rope_kv_write_partials: bad cache geometry");
  }
  if (n_tokens == 0) return 0;
  int px = 1;
  while (px < head_dim / 8) px <<= 1;
  int py = 256 / px;
  if (py < 1) py = 1;
  if (py > n_q_heads + n_kv_heads) py = n_q_heads + n_kv_heads;
  bf16_t* q = (bf16_t*)qkv;
  bf16_t* k = q + (size_t)n_q_heads * head_dim;
  bf16_t* v = k + (size_t)n_kv_heads * head_dim;
  const int gy = n_tokens >= 1024 ? 1 : (n_q_heads + n_kv_heads + py - 1) / py;
  hipLaunchKernelGGL(rope_kv_write_bf16x8_kernel<true>, dim3(n_tokens, gy), dim3(px, py), 0, stream, q, qkv_stride, k, qkv_stride, v,
                     qkv_stride, positions, seq_of_token, inv_freq, (bf16_t*)cache, block_table, table_width, page_size,
                     num_pages, n_q_heads, n_kv_heads, head_dim, partials, n_partials, partial_stride);
  return cwm_launch_status("rope_kv_write_partials");
}
