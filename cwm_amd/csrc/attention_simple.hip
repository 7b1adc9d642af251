// Paged causal attention with grouped heads and an optional sliding window: the
// plain kernel.  Keys are read from the paged cache through the sequence's block
// table; scores, softmax and the output sum are float32 for either storage type.
// It takes any head size up to 256, any page size and any head counts, and is the
// kernel of the float32 path.
//
// Formula (cwm/fastgen/forward.py:638-655): query at absolute position p of its
// sequence reads keys j with max(0, p - window_left) <= j <= p (window_left < 0:
// from 0); s_j = (q . k_j) * scale; o = sum_j softmax(s)_j v_j; query head h uses
// key/value head h / (n_q_heads / n_kv_heads).
//
// One block of four wavefronts per (token, key/value head, up to 8 of its query heads,
// segment of the keys): a key and a value are loaded once and used for all the block's
// query heads.  A token's keys are cut into segments by a rule of their number alone
// (one segment up to 2,048 keys, then ceil(n / 1,024) segments, at most 16, of equal
// length in chunks of 64: a window of 8,191 keys is read by eight blocks); the wavefronts of a block take the segment's chunks of 64
// keys in turn (scores and softmax: a lane per key; values: a lane per dimension) and join
// their results at the end in the order of the wavefronts; the segments of a token leave partial results (maximum, sum,
// unnormalised output) that a second kernel joins in the order of the segments.
//
// The order of every sum depends only on the token's own position and the window, so
// the result for a token is the same bits whatever else is in the batch and however
// the sequence was cut into steps.
#include "common.h"

CWM_DEFINE_ERROR_API

#define SIMPLE_MAX_HEAD_DIM 256
#define SIMPLE_WAVES 4      // wavefronts of a block: they take the segment's chunks of keys in turn
#define SIMPLE_HEADS 8      // query heads of one key/value head that a block serves at once
#define SIMPLE_SEGMENT 2048 // keys up to which a token has one segment
#define SIMPLE_SEGMENT_LONG 1024 // keys of a segment, about, of a token with more (until there are SIMPLE_MAX_SEGMENTS)
#define SIMPLE_MAX_SEGMENTS 16
#ifndef SIMPLE_K_ROUND
#define SIMPLE_K_ROUND 8     // 16-byte loads of a key's row that are in flight together
#endif
#ifndef SIMPLE_V_ROUND
#define SIMPLE_V_ROUND 5     // blocks of 8 values whose loads are in flight together
#endif
#define SIMPLE_D_REGS (SIMPLE_MAX_HEAD_DIM / CWM_WAVE)

extern "C" int cwm_attention_simple_max_segments() { return SIMPLE_MAX_SEGMENTS; }
extern "C" int cwm_attention_simple_segment_keys() { return SIMPLE_SEGMENT; }

// what one lane of a wavefront wrote to LDS, the wavefront's other lanes read after this
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// segments of a token that reads n_keys keys, and their length (a multiple of 64)
__device__ __forceinline__ int segments_of(int n_keys, int& seg_len) {
  int n_seg = 1;
  if (n_keys > SIMPLE_SEGMENT) n_seg = min(SIMPLE_MAX_SEGMENTS, (n_keys + SIMPLE_SEGMENT_LONG - 1) / SIMPLE_SEGMENT_LONG);
  seg_len = ((n_keys + n_seg - 1) / n_seg + CWM_WAVE - 1) / CWM_WAVE * CWM_WAVE;
  return n_seg;
}

// partial result of (token, query head, segment): [head_dim] unnormalised output, then maximum and sum
#define PARTIAL_STRIDE(hd) ((hd) + 2)

// HEADS: query heads a block serves (at most HEADS); D_REGS: dimensions of a head per lane (head sizes up to
// 64 * D_REGS).  The arithmetic is the same for every pair; smaller ones leave registers for more wavefronts.
template <typename T, int HEADS, int D_REGS>
__global__ void __launch_bounds__(SIMPLE_WAVES * CWM_WAVE)
attention_simple_kernel(const T* __restrict__ q, long q_stride, T* __restrict__ out, long out_stride,
                        const T* __restrict__ cache, const int* __restrict__ block_table, int table_width,
                        const int* __restrict__ positions, const int* __restrict__ seq_of_token, float* __restrict__ partial,
                        int n_q_heads, int n_kv_heads, int head_groups, int head_dim, int page_size, int num_pages,
                        int window_left, float scale) {
  __shared__ __attribute__((aligned(16))) float qs[HEADS][D_REGS * CWM_WAVE];
  // probabilities of a chunk, key jj at [in0 + jj] (in0: the first key's place in its block of 8 values), so that the
  // eight of a block lie at a multiple of 8
  __shared__ __attribute__((aligned(16))) float ps_all[SIMPLE_WAVES][HEADS][CWM_WAVE + 8];
  __shared__ long long voff_all[SIMPLE_WAVES][CWM_WAVE];
  __shared__ float part_m[SIMPLE_WAVES][HEADS], part_l[SIMPLE_WAVES][HEADS];
  __shared__ float part_o[SIMPLE_WAVES][HEADS][D_REGS * CWM_WAVE];

  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const int wave = threadIdx.x / CWM_WAVE;
  const int group = n_q_heads / n_kv_heads;
  int id = blockIdx.x;
  const int hg = id % head_groups;
  id /= head_groups;
  const int g = id % n_kv_heads;
  const int t = id / n_kv_heads;
  const int seg = blockIdx.y;
  const int h0 = g * group + hg * SIMPLE_HEADS;             // the block's first query head
  const int nh = min(SIMPLE_HEADS, group - hg * SIMPLE_HEADS);  // and how many it serves
  const int p = positions[t];
  const int b = seq_of_token[t];
  const int start = window_left >= 0 ? max(0, p - window_left) : 0;
  int seg_len;
  const int n_seg = segments_of(p - start + 1, seg_len);
  if (seg >= n_seg) return;
  if (n_seg > (int)gridDim.y || (n_seg > 1 && partial == nullptr)) {
    // the caller's `max_keys` was below what this token reads: the launch has no block (or no scratch) for
    // some of its segments.  Its rows come out NaN; nothing else is touched.
    if (seg == 0)
      for (int e = threadIdx.x; e < nh * head_dim; e += SIMPLE_WAVES * CWM_WAVE)
        Elem<T>::store(out + (size_t)t * out_stride + (size_t)h0 * head_dim + e, __uint_as_float(0x7fc00000u));
    return;
  }
  const int k0 = start + seg * seg_len;
  const int k1 = min(p + 1, k0 + seg_len);  // exclusive

  const size_t plane = (size_t)n_kv_heads * page_size * head_dim;
  const int v_block = (page_size % 8 == 0) ? 8 : page_size;
  const float neg_inf = -__builtin_inff();
  const float nan = __uint_as_float(0x7fc00000u);
  // float32 rows of keys and blocks of values can be read 16 bytes at a time
  const bool vec4 = head_dim % 4 == 0 && ((uintptr_t)cache % 16) == 0;

  for (int e = threadIdx.x; e < nh * head_dim; e += SIMPLE_WAVES * CWM_WAVE) {
    const int h = e / head_dim, d = e - h * head_dim;
    qs[h][d] = Elem<T>::load(q + (size_t)t * q_stride + (size_t)(h0 + h) * head_dim + d);
  }
  __syncthreads();

  float* ps = &ps_all[wave][0][0];
  long long* voff = voff_all[wave];
  float m[HEADS], l[HEADS];
  float o[HEADS][D_REGS];
#pragma unroll
  for (int h = 0; h < HEADS; ++h) {
    m[h] = neg_inf;
    l[h] = 0.f;
#pragma unroll
    for (int r = 0; r < D_REGS; ++r) o[h][r] = 0.f;
  }

  // wavefront w takes the chunks of 64 keys w, w + SIMPLE_WAVES, ... of the segment
  for (int base = k0 + wave * CWM_WAVE; base < k1; base += SIMPLE_WAVES * CWM_WAVE) {
    const int j = base + lane;
    const bool valid = j < k1;
    const int n = min(CWM_WAVE, k1 - base);
    const int in0 = base & 7;  // the first key's place in its block of 8 values
    float s[HEADS];
#pragma unroll
    for (int h = 0; h < HEADS; ++h) s[h] = neg_inf;
    long long vo = -1;
    if (valid) {
      const int lp = j / page_size;
      const int slot = j - lp * page_size;
      const int page = lp < table_width ? block_table[(size_t)b * table_width + lp] : -1;
      if (page < 0 || page >= num_pages) {
#pragma unroll
        for (int h = 0; h < HEADS; ++h) s[h] = nan;  // a key that should be there has no page: make it show
      } else {
        const T* krow = cache + (size_t)page * 2 * plane + ((size_t)g * page_size + slot) * head_dim;
        float dot[HEADS];
#pragma unroll
        for (int h = 0; h < HEADS; ++h) dot[h] = 0.f;
        if (sizeof(T) == 4 && vec4) {
          // 4 * SIMPLE_K_ROUND values per round of loads; every sum keeps the order d = 0, 1, 2, ...
          int d = 0;
          for (; d + 4 * SIMPLE_K_ROUND <= head_dim; d += 4 * SIMPLE_K_ROUND) {
            float4 kv[SIMPLE_K_ROUND];
#pragma unroll
            for (int u = 0; u < SIMPLE_K_ROUND; ++u) kv[u] = *(const float4*)((const float*)krow + d + 4 * u);
#pragma unroll
            for (int u = 0; u < SIMPLE_K_ROUND; ++u) {
#pragma unroll
              for (int h = 0; h < HEADS; ++h) {
                if (h < nh) {
                  const float4 qv = *(const float4*)(&qs[h][d + 4 * u]);
                  dot[h] = fmaf(qv.x, kv[u].x, dot[h]);
                  dot[h] = fmaf(qv.y, kv[u].y, dot[h]);
                  dot[h] = fmaf(qv.z, kv[u].z, dot[h]);
                  dot[h] = fmaf(qv.w, kv[u].w, dot[h]);
                }
              }
            }
          }
          for (; d < head_dim; d += 4) {
            const float4 kv = *(const float4*)((const float*)krow + d);
#pragma unroll
            for (int h = 0; h < HEADS; ++h) {
              if (h < nh) {
                const float4 qv = *(const float4*)(&qs[h][d]);
                dot[h] = fmaf(qv.x, kv.x, dot[h]);
                dot[h] = fmaf(qv.y, kv.y, dot[h]);
                dot[h] = fmaf(qv.z, kv.z, dot[h]);
                dot[h] = fmaf(qv.w, kv.w, dot[h]);
              }
            }
          }
        } else {
          for (int d = 0; d < head_dim; ++d) {
            const float kd = Elem<T>::load(krow + d);
#pragma unroll
            for (int h = 0; h < HEADS; ++h)
              if (h < nh) dot[h] = fmaf(qs[h][d], kd, dot[h]);
          }
        }
#pragma unroll
        for (int h = 0; h < HEADS; ++h) s[h] = dot[h] * scale;
        // values: blocks of v_block keys, [slot / v_block][dim][slot % v_block]
        vo = (long long)((size_t)page * 2 * plane + plane + (size_t)g * head_dim * page_size +
                         (size_t)(slot / v_block) * head_dim * v_block + slot % v_block);
      }
    }
    float alpha[HEADS];
#pragma unroll
    for (int h = 0; h < HEADS; ++h) {
      if (h < nh) {
        const float mx = wave_max(s[h]);
        const float m_new = fmaxf(m[h], mx);
        alpha[h] = (m[h] == neg_inf) ? 0.f : expf(m[h] - m_new);
        const float pj = valid ? expf(s[h] - m_new) : 0.f;
        l[h] = l[h] * alpha[h] + wave_sum(pj);
        ps[h * (CWM_WAVE + 8) + in0 + lane] = pj;
        m[h] = m_new;
      } else {
        alpha[h] = 0.f;
      }
    }
    voff[lane] = vo;
    wave_sync();  // the wavefront's own lanes read these next
#pragma unroll
    for (int r = 0; r < D_REGS; ++r) {
      const int d = lane + r * CWM_WAVE;
      if (d < head_dim) {
        float acc[HEADS];
#pragma unroll
        for (int h = 0; h < HEADS; ++h) acc[h] = o[h][r] * alpha[h];
        if (sizeof(T) == 4 && vec4 && v_block == 8) {
          // the eight keys of a block of values lie side by side for one dimension: two loads serve up to
          // eight keys.  The chunk's 64 keys lie in at most nine such blocks; the loads of several are issued
          // before the first is used; every sum keeps the order of the keys.
          // (SIMPLE_V_ROUND blocks a round of loads: the registers that nine would take cost a wavefront per SIMD)
#pragma unroll
          for (int b0 = 0; b0 < 9; b0 += SIMPLE_V_ROUND) {
            float4 lo[SIMPLE_V_ROUND], hi[SIMPLE_V_ROUND];
#pragma unroll
            for (int u = 0; u < SIMPLE_V_ROUND; ++u) {
              const int blk = b0 + u;
              const int jj = max(0, 8 * blk - in0);  // the block's first key of this chunk
              lo[u] = hi[u] = make_float4(nan, nan, nan, nan);
              if (blk < 9 && jj < n && (blk < 8 || in0 > 0)) {
                const long long off = voff[jj];
                if (off >= 0) {
                  const float* vb = (const float*)cache + (off - ((base + jj) & 7)) + (size_t)d * 8;
                  lo[u] = *(const float4*)vb;
                  hi[u] = *(const float4*)(vb + 4);
                }
              }
            }
#pragma unroll
            for (int u = 0; u < SIMPLE_V_ROUND; ++u) {
              const int blk = b0 + u;
              if (blk >= 9 || 8 * blk - in0 >= n) break;
              const float vv[8] = {lo[u].x, lo[u].y, lo[u].z, lo[u].w, hi[u].x, hi[u].y, hi[u].z, hi[u].w};
              float pp[HEADS][8];
#pragma unroll
              for (int h = 0; h < HEADS; ++h) {
                if (h < nh) {
                  const float4 pl = *(const float4*)(&ps[h * (CWM_WAVE + 8) + 8 * blk]);
                  const float4 ph = *(const float4*)(&ps[h * (CWM_WAVE + 8) + 8 * blk + 4]);
                  pp[h][0] = pl.x; pp[h][1] = pl.y; pp[h][2] = pl.z; pp[h][3] = pl.w;
                  pp[h][4] = ph.x; pp[h][5] = ph.y; pp[h][6] = ph.z; pp[h][7] = ph.w;
                }
              }
#pragma unroll
              for (int x = 0; x < 8; ++x) {
                const int jj = 8 * blk + x - in0;
                if (jj >= 0 && jj < n) {
#pragma unroll
                  for (int h = 0; h < HEADS; ++h)
                    if (h < nh) acc[h] = fmaf(pp[h][x], vv[x], acc[h]);
                }
              }
            }
          }
        } else {
          for (int jj = 0; jj < n; ++jj) {
            const long long off = voff[jj];
            const float vv = off >= 0 ? Elem<T>::load(cache + off + (size_t)d * v_block) : nan;
#pragma unroll
            for (int h = 0; h < HEADS; ++h)
              if (h < nh) acc[h] = fmaf(ps[h * (CWM_WAVE + 8) + in0 + jj], vv, acc[h]);
          }
        }
#pragma unroll
        for (int h = 0; h < HEADS; ++h) o[h][r] = acc[h];
      }
    }
    wave_sync();
  }

  // the wavefronts' results, joined in the order of the wavefronts
#pragma unroll
  for (int h = 0; h < HEADS; ++h) {
    if (h < nh) {
      if (lane == 0) {
        part_m[wave][h] = m[h];
        part_l[wave][h] = l[h];
      }
#pragma unroll
      for (int r = 0; r < D_REGS; ++r) {
        const int d = lane + r * CWM_WAVE;
        if (d < head_dim) part_o[wave][h][d] = o[h][r];
      }
    }
  }
  __syncthreads();
  // wavefront w finishes heads w, w + SIMPLE_WAVES, ...
  for (int h = wave; h < nh; h += SIMPLE_WAVES) {
    float m_all = part_m[0][h];
#pragma unroll
    for (int w = 1; w < SIMPLE_WAVES; ++w) m_all = fmaxf(m_all, part_m[w][h]);
    float weight[SIMPLE_WAVES];
    float l_all = 0.f;
#pragma unroll
    for (int w = 0; w < SIMPLE_WAVES; ++w) {
      weight[w] = (part_m[w][h] == neg_inf) ? 0.f : expf(part_m[w][h] - m_all);  // -inf: that wavefront had no chunk
      l_all += part_l[w][h] * weight[w];
    }
    T* orow = out + (size_t)t * out_stride + (size_t)(h0 + h) * head_dim;
    float* prow = n_seg > 1 ? partial + (((size_t)t * n_q_heads + h0 + h) * SIMPLE_MAX_SEGMENTS + seg) * PARTIAL_STRIDE(head_dim) : nullptr;
#pragma unroll
    for (int r = 0; r < D_REGS; ++r) {
      const int d = lane + r * CWM_WAVE;
      if (d < head_dim) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < SIMPLE_WAVES; ++w) sum += part_o[w][h][d] * weight[w];
        if (n_seg > 1)
          prow[d] = sum;
        else
          Elem<T>::store(orow + d, sum / l_all);
      }
    }
    if (n_seg > 1 && lane == 0) {
      prow[head_dim] = m_all;
      prow[head_dim + 1] = l_all;
    }
  }
}

// Joins the segments of the tokens that have several, in the order of the segments.  One wavefront
// per (token, query head).
template <typename T>
__global__ void __launch_bounds__(CWM_WAVE)
attention_simple_join_kernel(T* __restrict__ out, long out_stride, const float* __restrict__ partial,
                             const int* __restrict__ positions, int n_q_heads, int head_dim, int window_left,
                             int max_segments) {
  const int t = blockIdx.x / n_q_heads;
  const int h = blockIdx.x - t * n_q_heads;
  const int lane = threadIdx.x;
  const int p = positions[t];
  const int start = window_left >= 0 ? max(0, p - window_left) : 0;
  int seg_len;
  const int n_seg = segments_of(p - start + 1, seg_len);
  if (n_seg <= 1 || n_seg > max_segments) return;  // more than the launch had room for: the rows are NaN already
  const float neg_inf = -__builtin_inff();
  const float* base = partial + (((size_t)t * n_q_heads + h) * SIMPLE_MAX_SEGMENTS) * PARTIAL_STRIDE(head_dim);
  float m_all = neg_inf;
  for (int s = 0; s < n_seg; ++s) m_all = fmaxf(m_all, base[(size_t)s * PARTIAL_STRIDE(head_dim) + head_dim]);
  float l_all = 0.f;
  float o[SIMPLE_D_REGS];
#pragma unroll
  for (int r = 0; r < SIMPLE_D_REGS; ++r) o[r] = 0.f;
  for (int s = 0; s < n_seg; ++s) {
    const float* prow = base + (size_t)s * PARTIAL_STRIDE(head_dim);
    const float ms = prow[head_dim];
    const float weight = (ms == neg_inf) ? 0.f : expf(ms - m_all);
    l_all += prow[head_dim + 1] * weight;
#pragma unroll
    for (int r = 0; r < SIMPLE_D_REGS; ++r) {
      const int d = lane + r * CWM_WAVE;
      if (d < head_dim) o[r] += prow[d] * weight;
    }
  }
  T* orow = out + (size_t)t * out_stride + (size_t)h * head_dim;
#pragma unroll
  for (int r = 0; r < SIMPLE_D_REGS; ++r) {
    const int d = lane + r * CWM_WAVE;
    if (d < head_dim) Elem<T>::store(orow + d, o[r] / l_all);
  }
}

// `max_keys`: the most keys that any token of the call reads (its position + 1, or the window if that
// is less); `partial`: float32 scratch of n_tokens * n_q_heads * 16 * (head_dim + 2) values, needed
// (and touched) only if max_keys exceeds 2,048.  A token that reads more keys than `max_keys` says has no
// place for its segments' results: its rows of `out` are NaN and every kernel ends normally.
extern "C" int cwm_attention_simple(const void* q, long q_stride, void* out, long out_stride, const void* cache,
                                    int dtype, const int* block_table, int table_width, const int* positions,
                                    const int* seq_of_token, int n_tokens, int n_q_heads, int n_kv_heads,
                                    int head_dim, int page_size, int num_pages, int window_left, float scale,
                                    int max_keys, float* partial, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0, "attention: negative token count");
  CWM_REQUIRE(head_dim > 0 && head_dim <= SIMPLE_MAX_HEAD_DIM, "attention: head_dim %d is outside 1..%d", head_dim,
              SIMPLE_MAX_HEAD_DIM);
  CWM_REQUIRE(n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0,
              "attention: %d query heads do not divide into %d key/value heads", n_q_heads, n_kv_heads);
  CWM_REQUIRE(page_size > 0 && num_pages > 0 && table_width > 0, "attention: bad cache geometry");
  CWM_REQUIRE(max_keys >= 1, "attention: max_keys must be at least 1");
  if (n_tokens == 0) return 0;
  int max_segments = 1;
  if (max_keys > SIMPLE_SEGMENT) max_segments = (max_keys + SIMPLE_SEGMENT_LONG - 1) / SIMPLE_SEGMENT_LONG;  // as segments_of
  if (max_segments > SIMPLE_MAX_SEGMENTS) max_segments = SIMPLE_MAX_SEGMENTS;
  CWM_REQUIRE(max_segments == 1 || partial != nullptr, "attention: more than %d keys need the scratch for partial results",
              SIMPLE_SEGMENT);
  const int group = n_q_heads / n_kv_heads;
  const int head_groups = (group + SIMPLE_HEADS - 1) / SIMPLE_HEADS;
  const long long blocks = (long long)n_tokens * n_kv_heads * head_groups;
  CWM_REQUIRE(blocks <= 0x7fffffffLL, "attention: too many (token, head) pairs: %lld", blocks);
  const long long join_blocks = (long long)n_tokens * n_q_heads;
  CWM_REQUIRE(join_blocks <= 0x7fffffffLL, "attention: too many (token, head) pairs: %lld", join_blocks);
  dim3 grid((unsigned)blocks, (unsigned)max_segments);
  if (dtype == CWM_F32) {
    // the smallest block shape that holds the heads of a group and the head size
    const int heads = group < SIMPLE_HEADS ? group : SIMPLE_HEADS;
#define CWM_LAUNCH_SIMPLE(HEADS, D_REGS)                                                                                   \
  hipLaunchKernelGGL((attention_simple_kernel<float, HEADS, D_REGS>), grid, dim3(SIMPLE_WAVES * CWM_WAVE), 0, stream,     \
                     (const float*)q, q_stride, (float*)out, out_stride, (const float*)cache, block_table, table_width,   \
                     positions, seq_of_token, partial, n_q_heads, n_kv_heads, head_groups, head_dim, page_size, num_pages, \
                     window_left, scale)
#define CWM_LAUNCH_SIMPLE_HEADS(D_REGS)   \
  do {                                    \
    if (heads <= 2)                       \
      CWM_LAUNCH_SIMPLE(2, D_REGS);       \
    else if (heads <= 4)                  \
      CWM_LAUNCH_SIMPLE(4, D_REGS);       \
    else if (heads <= 6)                  \
      CWM_LAUNCH_SIMPLE(6, D_REGS);       \
    else                                  \
      CWM_LAUNCH_SIMPLE(SIMPLE_HEADS, D_REGS); \
  } while (0)
    if (head_dim <= CWM_WAVE)
      CWM_LAUNCH_SIMPLE_HEADS(1);
    else if (head_dim <= 2 * CWM_WAVE)
      CWM_LAUNCH_SIMPLE_HEADS(2);
    else
      CWM_LAUNCH_SIMPLE_HEADS(SIMPLE_D_REGS);
#undef CWM_LAUNCH_SIMPLE_HEADS
#undef CWM_LAUNCH_SIMPLE
    if (max_segments > 1)
      hipLaunchKernelGGL(attention_simple_join_kernel<float>, dim3((unsigned)join_blocks), dim3(CWM_WAVE), 0, stream,
                         (float*)out, out_stride, (const float*)partial, positions, n_q_heads, head_dim, window_left, max_segments);
  } else if (dtype == CWM_BF16) {
    hipLaunchKernelGGL((attention_simple_kernel<bf16_t, SIMPLE_HEADS, SIMPLE_D_REGS>), grid, dim3(SIMPLE_WAVES * CWM_WAVE), 0, stream, (const bf16_t*)q,
                       q_stride, (bf16_t*)out, out_stride, (const bf16_t*)cache, block_table, table_width, positions,
                       seq_of_token, partial, n_q_heads, n_kv_heads, head_groups, head_dim, page_size, num_pages, window_left,
                       scale);
    if (max_segments > 1)
      hipLaunchKernelGGL(attention_simple_join_kernel<bf16_t>, dim3((unsigned)join_blocks), dim3(CWM_WAVE), 0, stream,
                         (bf16_t*)out, out_stride, (const float*)partial, positions, n_q_heads, head_dim, window_left, max_segments);
  } else {
    return cwm_fail("attention: unknown dtype %d", dtype);
  }
  return cwm_launch_status("attention_simple");
}
