// Row-wise kernels of the decoder: token embedding gather, residual-add fused with
// RMSNorm, and SiLU(gate) * up.  All arithmetic is float32; storage types are
// chosen per argument (float32 or bfloat16).
//
// Formulas: embedding cwm/fastgen/forward.py:543-546; RMSNorm
// cwm/fastgen/kernels/rmsnorm.py:34-61; SiLU * up cwm/fastgen/forward.py:781.
#include "common.h"

CWM_DEFINE_ERROR_API

// ---- embedding: out[t, :] = scale * table[token[t], :] as float32 -------------- //
// (scale is 1 for the architecture of the reference; others multiply the embedding)
template <typename TW>
__global__ void embedding_kernel(float* __restrict__ out, const TW* __restrict__ table,
                                 const int* __restrict__ tokens, int dim, int vocab, float scale) {
  const int t = blockIdx.x;
  const int tok = tokens[t];
  float* dst = out + (size_t)t * dim;
  if (tok < 0 || tok >= vocab) {  // the host checks ids; never read outside the table
    for (int i = threadIdx.x; i < dim; i += blockDim.x) dst[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  const TW* src = table + (size_t)tok * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) dst[i] = scale * Elem<TW>::load(src + i);
}

extern "C" int cwm_embedding(void* out, const void* table, int table_dtype, const int* tokens,
                             int n_tokens, int dim, int vocab, float scale, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && dim > 0 && vocab > 0, "embedding: bad sizes T=%d D=%d V=%d", n_tokens, dim, vocab);
  if (n_tokens == 0) return 0;
  const int threads = dim >= 1024 ? 256 : (dim >= 256 ? 128 : 64);
  if (table_dtype == CWM_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream, (float*)out,
                       (const float*)table, tokens, dim, vocab, scale);
  else if (table_dtype == CWM_BF16)
    hipLaunchKernelGGL(embedding_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream, (float*)out,
                       (const bf16_t*)table, tokens, dim, vocab, scale);
  else
    return cwm_fail("embedding: unknown table dtype %d", table_dtype);
  return cwm_launch_status("embedding");
}

// ---- h += delta (float32), out = h * rsqrt(mean(h^2) + eps) * w ---------------- //
// One block per output row.  With `rows`, output row r is computed from source row
// rows[r] and h is not modified.
template <typename TD, typename TW, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_partials,
                                   long partial_stride, const TW* __restrict__ weight, TO* __restrict__ out,
                                   const int* __restrict__ rows, int dim, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* hrow = h + (size_t)src * dim;
  const TD* drow = delta ? delta + (size_t)src * dim : nullptr;
  const bool write_back = (delta != nullptr) && (rows == nullptr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    float v = hrow[i];
    if (drow) {
      for (int p = 0; p < n_partials; ++p) v += Elem<TD>::load(drow + (size_t)p * partial_stride + i);
      if (write_back) hrow[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(ss / (float)dim + eps);
  TO* orow = out + (size_t)r * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    float v = hrow[i];
    if (drow && !write_back)
      for (int p = 0; p < n_partials; ++p) v += Elem<TD>::load(drow + (size_t)p * partial_stride + i);
    Elem<TO>::store(orow + i, v * rstd * Elem<TW>::load(weight + i));
  }
}

// The same for rows that fit in registers (dim % 4 == 0, dim <= 4 * CHUNKS * threads):
// every load of a row is issued at once, the row is read once and never re-read.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 x = *(const float4*)p;
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Vec4<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *(const uint2*)p;
    v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    uint2 x;
    x.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
    x.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
    *(uint2*)p = x;
  }
};

template <typename TD, typename TW, typename TO, int CHUNKS>
__global__ void add_rmsnorm_regs_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_partials,
                                        long partial_stride, const TW* __restrict__ weight, TO* __restrict__ out,
                                        const int* __restrict__ rows, int dim, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* hrow = h + (size_t)src * dim;
  const TD* drow = delta ? delta + (size_t)src * dim : nullptr;
  const bool write_back = (delta != nullptr) && (rows == nullptr);
  const int n_chunks = dim >> 2;
  float v[CHUNKS][4], w[CHUNKS][4];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int chunk = threadIdx.x + c * blockDim.x;
    if (chunk < n_chunks) {
      Vec4<float>::load(hrow + 4 * chunk, v[c]);
      Vec4<TW>::load(weight + 4 * chunk, w[c]);
      if (drow) {
        // four partial sums in flight at a time (a fifth would wait for the first otherwise); what lies
        // past the last one is loaded again from the last and not added; the order of the sum stays p = 0, 1, ...
        if (n_partials == 1) {
          float d[4];
          Vec4<TD>::load(drow + 4 * chunk, d);
#pragma unroll
          for (int i = 0; i < 4; ++i) v[c][i] += d[i];
        } else
        for (int p = 0; p < n_partials; p += 4) {
          float d[4][4];
#pragma unroll
          for (int u = 0; u < 4; ++u) Vec4<TD>::load(drow + (size_t)min(p + u, n_partials - 1) * partial_stride + 4 * chunk, d[u]);
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const float keep = p + u < n_partials ? 1.0f : 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[c][i] += keep * d[u][i];
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[c][i] = w[c][i] = 0.f;
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int chunk = threadIdx.x + c * blockDim.x;
    if (write_back && chunk < n_chunks) Vec4<float>::store(hrow + 4 * chunk, v[c]);
#pragma unroll
    for (int i = 0; i < 4; ++i) ss += v[c][i] * v[c][i];
  }
  ss = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(ss / (float)dim + eps);
  TO* orow = out + (size_t)r * dim;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int chunk = threadIdx.x + c * blockDim.x;
    if (chunk < n_chunks) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = v[c][i] * rstd * w[c][i];
      Vec4<TO>::store(orow + 4 * chunk, y);
    }
  }
}

template <typename TD, typename TW, typename TO>
static void launch_add_rmsnorm(void* h, const void* delta, int n_partials, long partial_stride, const void* w, void* out,
                               const int* rows, int n_out, int dim, float eps, hipStream_t stream) {
  const int n_chunks = dim / 4;
  if (dim % 4 == 0 && n_chunks <= 4 * 512) {
    // all pointers are rows of contiguous tensors whose row length is a multiple of 4: 16-byte aligned loads
    int threads = 64;
    while (threads < 512 && threads * 4 < n_chunks) threads *= 2;
    const int chunks = (n_chunks + threads - 1) / threads;
    auto go = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(n_out), dim3(threads), 0, stream, (float*)h, (const TD*)delta, n_partials,
                         partial_stride, (const TW*)w, (TO*)out, rows, dim, eps);
    };
    if (chunks <= 1) go(add_rmsnorm_regs_kernel<TD, TW, TO, 1>);
    else if (chunks <= 2) go(add_rmsnorm_regs_kernel<TD, TW, TO, 2>);
    else if (chunks <= 3) go(add_rmsnorm_regs_kernel<TD, TW, TO, 3>);
    else go(add_rmsnorm_regs_kernel<TD, TW, TO, 4>);
    return;
  }
  const int threads = dim >= 2048 ? 512 : (dim >= 512 ? 256 : (dim >= 128 ? 128 : 64));
  hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TW, TO>), dim3(n_out), dim3(threads), 0, stream, (float*)h,
                     (const TD*)delta, n_partials, partial_stride, (const TW*)w, (TO*)out, rows, dim, eps);
}

extern "C" int cwm_add_rmsnorm(void* h, const void* delta, int delta_dtype, int n_partials, long partial_stride,
                               const void* weight, int weight_dtype, void* out, int out_dtype, const int* rows,
                               int n_out, int dim, float eps, hipStream_t stream) {
  CWM_REQUIRE(n_out >= 0 && dim > 0, "add_rmsnorm: bad sizes rows=%d D=%d", n_out, dim);
  CWM_REQUIRE(n_partials >= 1 && (n_partials == 1 || delta_dtype == CWM_F32), "add_rmsnorm: partial sums must be float32");
  CWM_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be positive");
  if (n_out == 0) return 0;
  if (!delta) delta_dtype = CWM_F32;
  const int key = (delta_dtype << 2) | (weight_dtype << 1) | out_dtype;
  switch (key) {
    case 0: launch_add_rmsnorm<float, float, float>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    case 1: launch_add_rmsnorm<float, float, bf16_t>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    case 2: launch_add_rmsnorm<float, bf16_t, float>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    case 3: launch_add_rmsnorm<float, bf16_t, bf16_t>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    case 4: launch_add_rmsnorm<bf16_t, float, float>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    case 5: launch_add_rmsnorm<bf16_t, float, bf16_t>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    case 6: launch_add_rmsnorm<bf16_t, bf16_t, float>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    case 7: launch_add_rmsnorm<bf16_t, bf16_t, bf16_t>(h, delta, n_partials, partial_stride, weight, out, rows, n_out, dim, eps, stream); break;
    default: return cwm_fail("add_rmsnorm: unknown dtypes delta=%d weight=%d out=%d", delta_dtype, weight_dtype, out_dtype);
  }
  return cwm_launch_status("add_rmsnorm");
}

// ---- out[t, f] = silu(gate[t, f]) * up[t, f] ------------------------------------ //
// Row t of x holds 2F values: gate[f] at f and up[f] at F + f, or, with `grouped`, gate and up
// in alternating groups of 8 (gate[f] at 16 * (f / 8) + f % 8, up[f] 8 further), the order in
// which a product with row-interleaved gate/up weights delivers them.
template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ x, int hidden, size_t total, int grouped) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    const size_t t = idx / hidden;
    const int f = (int)(idx - t * hidden);
    const T* row = x + t * 2 * (size_t)hidden;
    const int at = grouped ? 16 * (f >> 3) + (f & 7) : f;
    const float g = Elem<T>::load(row + at);
    const float u = Elem<T>::load(row + at + (grouped ? 8 : hidden));
    const float s = g / (1.0f + expf(-g));
    Elem<T>::store(out + idx, s * u);
  }
}

// eight bfloat16 pairs per thread, 16-byte loads and stores (hidden % 8 == 0)
__global__ void silu_mul_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x, int hidden8, size_t total8,
                                       int grouped) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total8; idx += stride) {
    const size_t t = idx / hidden8;
    const int f8 = (int)(idx - t * hidden8);
    const bf16_t* row = x + t * 16 * (size_t)hidden8;
    const uint4 g = *(const uint4*)(row + (grouped ? 16 : 8) * f8);
    const uint4 u = *(const uint4*)(row + (grouped ? 16 * f8 + 8 : 8 * (size_t)hidden8 + 8 * f8));
    const uint32_t gi[4] = {g.x, g.y, g.z, g.w};
    const uint32_t ui[4] = {u.x, u.y, u.z, u.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float g0 = __uint_as_float(gi[i] << 16), g1 = __uint_as_float(gi[i] & 0xffff0000u);
      const float u0 = __uint_as_float(ui[i] << 16), u1 = __uint_as_float(ui[i] & 0xffff0000u);
      const float s0 = g0 / (1.0f + expf(-g0));
      const float s1 = g1 / (1.0f + expf(-g1));
      o[i] = (uint32_t)f32_to_bf16(s0 * u0) | ((uint32_t)f32_to_bf16(s1 * u1) << 16);
    }
    *(uint4*)(out + 8 * idx) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// The same from float32 partial sums x[p][t][2F] of a product whose K was split: the partials are
// added in order p = 0, 1, ..., the sums rounded to the output type (as the product would have
// stored them), then silu(gate) * up.  Four columns per thread (hidden % 4 == 0).
template <typename T>
__global__ void silu_mul_partials_kernel(T* __restrict__ out, const float* __restrict__ x, int n_partials, size_t part_stride,
                                         int hidden4, size_t total4, int grouped) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total4; idx += stride) {
    const size_t t = idx / hidden4;
    const int f4 = (int)(idx - t * hidden4);
    const float* row = x + t * 8 * (size_t)hidden4 + (grouped ? 16 * (f4 >> 1) + 4 * (f4 & 1) : 4 * f4);
    const size_t to_up = grouped ? 8 : 4 * (size_t)hidden4;
    float4 g = make_float4(0.f, 0.f, 0.f, 0.f), u = g;
    for (int p = 0; p < n_partials; ++p) {
      const float4 gp = *(const float4*)(row + p * part_stride);
      const float4 up = *(const float4*)(row + p * part_stride + to_up);
      g.x += gp.x; g.y += gp.y; g.z += gp.z; g.w += gp.w;
      u.x += up.x; u.y += up.y; u.z += up.z; u.w += up.w;
    }
    const float gs[4] = {g.x, g.y, g.z, g.w};
    const float us[4] = {u.x, u.y, u.z, u.w};
    T* o = out + 4 * idx;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      T gr, ur;
      Elem<T>::store(&gr, gs[i]);
      Elem<T>::store(&ur, us[i]);
      const float gv = Elem<T>::load(&gr), uv = Elem<T>::load(&ur);
      Elem<T>::store(o + i, gv / (1.0f + expf(-gv)) * uv);
    }
  }
}

extern "C" int cwm_silu_mul_partials(void* out, int out_dtype, const void* partials, int n_partials, int n_tokens, int hidden,
                                     int grouped, hipStream_t stream) {
  CWM_REQUIRE(!grouped || hidden % 8 == 0, "silu_mul_partials: groups of 8 need F=%d to be a multiple of 8", hidden);
  CWM_REQUIRE(n_tokens >= 0 && hidden > 0 && n_partials > 0, "silu_mul_partials: bad sizes P=%d T=%d F=%d", n_partials,
              n_tokens, hidden);
  CWM_REQUIRE(hidden % 4 == 0 && ((uintptr_t)partials % 16) == 0, "silu_mul_partials: F=%d must be a multiple of 4 and the "
              "partial sums 16-byte aligned", hidden);
  if (n_tokens == 0) return 0;
  const size_t total4 = (size_t)n_tokens * (hidden / 4);
  const size_t part_stride = (size_t)n_tokens * 2 * hidden;
  const int threads = 256;
  size_t blocks = (total4 + threads - 1) / threads;
  if (blocks > 16384) blocks = 16384;
  if (out_dtype == CWM_F32)
    hipLaunchKernelGGL(silu_mul_partials_kernel<float>, dim3((unsigned)blocks), dim3(threads), 0, stream, (float*)out,
                       (const float*)partials, n_partials, part_stride, hidden / 4, total4, grouped);
  else if (out_dtype == CWM_BF16)
    hipLaunchKernelGGL(silu_mul_partials_kernel<bf16_t>, dim3((unsigned)blocks), dim3(threads), 0, stream, (bf16_t*)out,
                       (const float*)partials, n_partials, part_stride, hidden / 4, total4, grouped);
  else
    return cwm_fail("silu_mul_partials: unknown dtype %d", out_dtype);
  return cwm_launch_status("silu_mul_partials");
}

extern "C" int cwm_silu_mul(void* out, const void* x, int dtype, int n_tokens, int hidden, int grouped, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && hidden > 0, "silu_mul: bad sizes T=%d F=%d", n_tokens, hidden);
  CWM_REQUIRE(!grouped || hidden % 8 == 0, "silu_mul: groups of 8 need F=%d to be a multiple of 8", hidden);
  if (n_tokens == 0) return 0;
  const size_t total = (size_t)n_tokens * hidden;
  const int threads = 256;
  if (dtype == CWM_BF16 && hidden % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    const size_t total8 = total / 8;
    size_t blocks = (total8 + threads - 1) / threads;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3((unsigned)blocks), dim3(threads), 0, stream, (bf16_t*)out,
                       (const bf16_t*)x, hidden / 8, total8, grouped);
    return cwm_launch_status("silu_mul");
  }
  size_t blocks = (total + threads - 1) / threads;
  if (blocks > 65536) blocks = 65536;
  if (dtype == CWM_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, dim3((unsigned)blocks), dim3(threads), 0, stream, (float*)out,
                       (const float*)x, hidden, total, grouped);
  else if (dtype == CWM_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, dim3((unsigned)blocks), dim3(threads), 0, stream, (bf16_t*)out,
                       (const bf16_t*)x, hidden, total, grouped);
  else
    return cwm_fail("silu_mul: unknown dtype %d", dtype);
  return cwm_launch_status("silu_mul");
}

// ---- out = sum over p of partials[p] (float32, in order) ----------------------- //
template <typename TO>
__global__ void sum_partials_kernel(TO* __restrict__ out, const float* __restrict__ partials, int n_partials, long count) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < count; i += stride) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += partials[(size_t)p * count + i];
    Elem<TO>::store(out + i, v);
  }
}

extern "C" int cwm_sum_partials(void* out, int out_dtype, const float* partials, int n_partials, long count,
                                hipStream_t stream) {
  CWM_REQUIRE(n_partials >= 1 && count >= 0, "sum_partials: bad sizes");
  if (count == 0) return 0;
  long blocks = (count + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (out_dtype == CWM_F32)
    hipLaunchKernelGGL(sum_partials_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, (float*)out, partials,
                       n_partials, count);
  else if (out_dtype == CWM_BF16)
    hipLaunchKernelGGL(sum_partials_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (bf16_t*)out, partials,
                       n_partials, count);
  else
    return cwm_fail("sum_partials: unknown dtype %d", out_dtype);
  return cwm_launch_status("sum_partials");
}
