// Paged causal attention on the matrix cores (bfloat16 storage, float32 softmax and
// accumulation), one kernel for prompt portions and for decoded tokens.  Compiled
// per head size: -DHEAD_DIM=<multiple of 16, at most 256>.
//
// Formula as cwm/fastgen/forward.py:638-655 (the reference calls FlashAttention-3
// there): query at position p reads keys max(0, p - window_left)..p of its sequence
// from the paged cache; scores (q . k) * scale; softmax; sum of values; query head
// h reads key/value head h / (Hq / Hkv).
//
// Decomposition.  For one sequence and one key/value head g the "rows" are the
// (new token, query head of g's group) pairs, row r = token (r / G), head g*G + r%G.
// A wavefront takes 16 consecutive rows and a range of keys (a work item built on
// the host): a decoded token's G heads are one tile and share every key and value
// load; a prompt portion is ceil(n*G/16) tiles.  Long key ranges of sequences with
// few rows are cut into chunks at fixed absolute positions; each chunk's wavefront
// writes a partial (max, sum, unnormalised output) and a second kernel merges them.
// The cut depends only on the sequence's own lengths, never on the rest of the
// batch, so a token's result does not depend on what it is batched with.
//
// Matrix-core layout (v_mfma_f32_16x16x32_bf16, 64 lanes, lane = 16*j + n):
//   S^T[key, row] = K[key, :] . Q[row, :]   A = K tile (lane: key n, dims 32s+8j..+7)
//                                            B = Q^T   (lane: row n, same dims)
//   result lane (row n, j) holds 4 keys per tile; two tiles whose A rows are picked
//   as key = 8*(m/4) + 4*tile + m%4 give that lane 8 consecutive keys 8j..8j+7,
//   which is exactly the B operand layout of
//   O^T[d, row] += V^T[d, key] . P^T[key, row]   A = V^T tile (lane: dim n, keys 8j..+7)
// so probabilities never move between lanes, and every operand load is 16
// contiguous bytes: keys are stored [slot][dim], values in blocks of 8 keys
// [slot / 8][dim][slot % 8].  The loop keeps the next tile's keys and this tile's
// values in flight while it computes.
//
// Matrix and vector instructions of one SIMD do not overlap on this chip (measured: their
// times add, also between wavefronts), so next to the matrix instructions the kernels'
// time is the count of vector instructions; v_exp_f32 costs four of them, v_max3_f32 and
// v_cvt_pk_bf16_f32 two.
#include "common.h"

CWM_DEFINE_ERROR_API

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
#if HEAD_DIM % 16 != 0 || HEAD_DIM > 256 || HEAD_DIM < 16
#error "HEAD_DIM must be a multiple of 16 between 16 and 256"
#endif

// dimension steps of 32 for Q K^T; if the head size leaves 16 over, the last step is
// half filled (lanes j >= 2 supply zeros), so that one instruction shape serves all
#define K32_STEPS ((HEAD_DIM + 31) / 32)
#define HALF_LAST_STEP ((HEAD_DIM % 32) != 0)
#define D_TILES (HEAD_DIM / 16)
#define WORK_INTS 6
#define PARTIAL_STRIDE (HEAD_DIM + 4)  // max and sum after the output; keeps rows 16-byte aligned

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) { return pack2_bf16(lo, hi); }
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// One row's share of a 32-key tile of scores: masks (only where a tile reaches past some
// row's keys), the probabilities as the matrix-core B operand, and the factor that rescales
// what was accumulated so far.  p = exp2(raw * c - m * c) is one fused multiply-add and one
// v_exp_f32 per score; a masked score is -inf, which the same two instructions turn into 0.
// m is a reference value, not the exact maximum: it moves (and everything accumulated is
// rescaled) only when the row's maximum has outgrown it by a factor of 256 in p; p <= 256 is
// exact enough in bfloat16 and float32 sums, and the final division by the sum of p (or the
// merge of partials, which takes any reference) undoes it.  Whether any row of the wavefront
// has outgrown its reference is one vote on each lane's own eight scores; only then are the
// lanes of a row compared (two exchanges through LDS) and the references moved, which after a
// sequence's first tiles almost never happens.  NEG_MC is -m * c, kept beside m.  VOTE = false
// compares the lanes in every tile, without a branch: the kernel for decoded tokens is bound
// by its loads, and a branch in its loop costs it more than the comparisons.
#define MAXIMUM(a, b) __builtin_elementwise_maximum(a, b)
#define SOFTMAX_TILE(VOTE, ST0, ST1, NEED_MASK, OK_EXPR, M_RUN, NEG_MC, L_RUN, ALPHA, PF)                    \
  {                                                                                                          \
    float rv[8] = {ST0[0], ST0[1], ST0[2], ST0[3], ST1[0], ST1[1], ST1[2], ST1[3]};                          \
    if (NEED_MASK) {                                                                                         \
      _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                                        \
        const int key = kt + 8 * j + e;                                                                      \
        rv[e] = (OK_EXPR) ? rv[e] : neg_inf;                                                                 \
      }                                                                                                      \
    }                                                                                                        \
    /* v_maximum3_f32 (no score is not a number: what a tile holds beyond a row's keys is -inf by now) */    \
    float tile_max = MAXIMUM(MAXIMUM(MAXIMUM(rv[0], rv[1]), MAXIMUM(rv[2], rv[3])), MAXIMUM(MAXIMUM(rv[4], rv[5]), MAXIMUM(rv[6], rv[7]))); \
    ALPHA = 1.0f;                                                                                            \
    if (!(VOTE) || __any(tile_max - M_RUN > lazy_raw)) {                                                     \
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));                                              \
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));                                              \
      const float m_top = fmaxf(M_RUN, tile_max);                                                            \
      const float m_new = (m_top - M_RUN > lazy_raw) ? m_top : M_RUN;                                        \
      const float neg_mc = (m_new == neg_inf) ? 0.f : -m_new * scale_log2e;                                  \
      ALPHA = __builtin_amdgcn_exp2f(fmaf(M_RUN, scale_log2e, neg_mc));                                      \
      L_RUN *= ALPHA;                                                                                        \
      M_RUN = m_new;                                                                                         \
      NEG_MC = neg_mc;                                                                                       \
    }                                                                                                        \
    float pv[8];                                                                                             \
    float psum = 0.f;                                                                                        \
    _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                                          \
      pv[e] = __builtin_amdgcn_exp2f(fmaf(rv[e], scale_log2e, NEG_MC));                                      \
      psum += pv[e];                                                                                         \
    }                                                                                                        \
    L_RUN += psum;                                                                                           \
    PF.u = make_uint4(pack_bf16(pv[0], pv[1]), pack_bf16(pv[2], pv[3]), pack_bf16(pv[4], pv[5]), pack_bf16(pv[6], pv[7])); \
  }

extern "C" int cwm_attention_mfma_head_dim() { return HEAD_DIM; }

__device__ __forceinline__ float not_a_number() { return __uint_as_float(0x7fc00000u); }

// Whether any key of [first_key, last_key] (a wavefront's span, the same for all its lanes) lies in a
// logical page whose table entry is no page of the pool: the lanes test the entries side by side.
__device__ __forceinline__ bool span_lacks_page(const int* __restrict__ table, int table_width, int num_pages,
                                                int page_size, int page_shift, int first_key, int last_key, int lane) {
  bool bad = false;
  if (last_key >= first_key && first_key >= 0) {
    const int lp_first = page_shift >= 0 ? (first_key >> page_shift) : (first_key / page_size);
    const int lp_last = page_shift >= 0 ? (last_key >> page_shift) : (last_key / page_size);
    for (int lp = lp_first + lane; lp <= lp_last; lp += 64) {
      const int page = lp < table_width ? table[lp] : -1;
      bad = bad || (unsigned)page >= (unsigned)num_pages;
    }
  }
  return __any(bad);
}

// work item: {sequence, first row, first key, end key (exclusive), partial slot or -1, unused}
// A block of four wavefronts (a team) per (work item, key/value head), on the 16 rows from the item's first
// row on: a decoded token's heads, or 16 rows of a short portion (sequences with many rows go to the kernel
// further down that shares keys and values through LDS).  Wavefront w takes the item's tiles of 32 keys
// w, w + 4, ... (so that the block reads consecutive memory), and the four combine their results through
// LDS at the end: four times the loads in flight for the same number of partial results, and a key range
// of up to 2,048 keys leaves no partial results at all.  Which wavefront takes which tile follows from the
// item alone, so a row's result still does not depend on the rest of the batch.
//
// A wavefront has its tile's values and the next tile's keys in flight while it computes; the loads of the
// next tile's keys stand in straight-line code (the last tile is processed apart), since a branch around them
// makes the compiler wait for every load in flight where the paths meet.  (Keys and values both a whole tile
// ahead, in two sets of registers, need more than 256 registers and spill.)
// PAGE32 (pages of a multiple of 32 keys): a tile lies in one page, whose number is read as a
// scalar; the scalar loads count apart from the vector loads, so looking up the next page does not wait for
// the loads in flight (a lookup by vector load, which returns in order behind them, would).  The values are
// read in whole cache lines, once: their loads are non-temporal and leave the caches alone (1,074 MB of a
// global layer at batch 8 and 32,768 tokens: 196 us before, 178 us with this alone).
#define TEAM 4
typedef const __attribute__((address_space(4))) int* scalar_ints;  // constant address space: a uniform index is read by a scalar load

template <bool PAGE32>
__global__ void __launch_bounds__(256, 2)
attention_mfma_kernel(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long out_stride,
                      const bf16_t* __restrict__ cache, const int* __restrict__ block_table, int table_width,
                      const int* __restrict__ cu_q, const int* __restrict__ kv_len, const int* __restrict__ work,
                      int n_work, float* __restrict__ partial, int n_q_heads, int n_kv_heads, int page_size,
                      int page_shift, int num_pages, int window_left, float scale_log2e) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int id = blockIdx.x;  // (item, key/value head): the same for the whole block
  const int item = id / n_kv_heads;
  const int g = id - item * n_kv_heads;
  if (item >= n_work) return;
  const int* w = work + (size_t)item * WORK_INTS;
  const int b = w[0];
  const int row0 = w[1];
  const int key_begin = w[2];
  const int key_end = w[3];
  const int slot = w[4];
  if (key_begin >= key_end) return;  // a null item: a list of a fixed length is filled up with them

  const int group = n_q_heads / n_kv_heads;
  const int q0 = cu_q[b];
  const int n_new = cu_q[b + 1] - q0;
  const int n_old = kv_len[b] - n_new;
  const int n_rows = n_new * group;

  const int n = lane & 15;  // row of the tile (B operands, results), key or dim of the tile (A operands)
  const int j = lane >> 4;

  // this lane's row
  const int r = row0 + n;
  const bool row_valid = r < n_rows;
  const int ti = row_valid ? r / group : 0;
  const int hq = g * group + (row_valid ? r - ti * group : 0);
  const int row_end = n_old + ti;  // last key the row may read
  const int row_start = window_left >= 0 ? max(0, row_end - window_left) : 0;
  // the span of keys that any row of the item reads (uniform): outside it values may be anything
  // (pages given back, slots never written) and are zeroed before use
  int lo_any = row_valid ? row_start : 0x7fffffff, hi_any = row_valid ? row_end : -1;
  // a tile every key of which every row reads needs no masks: from the latest first key to
  // the earliest last key over the rows (never, if some row of the tile does not exist)
  int lo_all = max(key_begin, row_valid ? row_start : 0x7fffffff), hi_all = min(key_end - 1, row_valid ? row_end : -1);
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) {
    lo_any = min(lo_any, __shfl_xor(lo_any, off, 64));
    hi_any = max(hi_any, __shfl_xor(hi_any, off, 64));
    lo_all = max(lo_all, __shfl_xor(lo_all, off, 64));
    hi_all = min(hi_all, __shfl_xor(hi_all, off, 64));
  }
  lo_any = max(lo_any, key_begin);
  hi_any = min(hi_any, key_end - 1);

  // queries: B operand, kept in registers for the whole loop
  Frag8 qf[K32_STEPS];
  {
    const bf16_t* qrow = q + (size_t)(q0 + ti) * q_stride + (size_t)hq * HEAD_DIM;
#pragma unroll
    for (int s = 0; s < K32_STEPS; ++s) {
      const bool filled = !(HALF_LAST_STEP && s == K32_STEPS - 1) || j < 2;
      if (row_valid && filled)
        qf[s].u = *(const uint4*)(qrow + 32 * s + 8 * j);
      else
        qf[s].u = make_uint4(0, 0, 0, 0);
    }
  }

  float4v acc[D_TILES];
  const float neg_inf = -__builtin_inff();
  const float lazy_raw = 8.0f / scale_log2e;  // 8 binary orders, in units of the raw scores
#pragma unroll
  for (int dt = 0; dt < D_TILES; ++dt) acc[dt] = (float4v){0.f, 0.f, 0.f, 0.f};
  float m_run = neg_inf, neg_mc_run = 0.f;
  float l_run = 0.f;  // this lane's share of the row's sum; the four lanes of a row are added at the end

  const size_t plane = (size_t)n_kv_heads * page_size * HEAD_DIM;
  const int* table = block_table + (size_t)b * table_width;
  const scalar_ints table_s = (scalar_ints)table;
  const bf16_t* kbase = cache + (size_t)g * page_size * HEAD_DIM;
  const bf16_t* vbase = cache + plane + (size_t)g * page_size * HEAD_DIM;
  // a key that some row reads must have a page: if its table entry is -1 or out of range the rows'
  // results are made NaN (the loads below then read page 0, so nothing faults)
  const bool page_missing = span_lacks_page(table, table_width, num_pages, page_size, page_shift, lo_any, hi_any, lane);

  // page of a key; keys outside [0, key_end) and slots without a page read page 0 and are masked
  auto page_of = [&](int key, int& slot_in_page) -> int {
    const int lp = page_shift >= 0 ? (key >> page_shift) : (key / page_size);
    slot_in_page = key - lp * page_size;
    int page = (key < key_end && lp < table_width) ? table[lp] : 0;
    return (page >= 0 && page < num_pages) ? page : 0;
  };
  // keys of the two 16-key tiles that this lane loads rows of: 8*(n/4) + 4*t + n%4
  const int krel0 = 8 * (n >> 2) + (n & 3);

  // page and first slot of the tile of 32 keys from `kt` on, for the lane's two key rows and its values
  auto locate = [&](int kt, int& p0, int& ks0, int& p1, int& ks1, int& vp, int& vs) {
    if (PAGE32) {
      const int lp = page_shift >= 0 ? (kt >> page_shift) : (kt / page_size);  // uniform
      const int first = kt - lp * page_size;
      int page = lp < table_width ? table_s[lp] : 0;
      page = (page >= 0 && page < num_pages) ? page : 0;
      p0 = p1 = vp = page;
      ks0 = first + krel0;
      ks1 = ks0 + 4;
      vs = first + 8 * j;
    } else {
      p0 = page_of(kt + krel0, ks0);
      p1 = page_of(kt + krel0 + 4, ks1);
      vp = page_of(kt + 8 * j, vs);
    }
  };
  // the loads of that tile's keys (A operands, two tiles of 16 keys) ...
  auto issue_keys = [&](Frag8 (&KF)[2][K32_STEPS], int kt) {
    int ks0, ks1, vs, p0, p1, vp;
    locate(kt, p0, ks0, p1, ks1, vp, vs);
    const bf16_t* kr0 = kbase + (size_t)p0 * 2 * plane + (size_t)ks0 * HEAD_DIM;
    const bf16_t* kr1 = kbase + (size_t)p1 * 2 * plane + (size_t)ks1 * HEAD_DIM;
#pragma unroll
    for (int s = 0; s < K32_STEPS; ++s) {
      const bool filled = !(HALF_LAST_STEP && s == K32_STEPS - 1) || j < 2;
      KF[0][s].u = filled ? *(const uint4*)(kr0 + 32 * s + 8 * j) : make_uint4(0, 0, 0, 0);
      KF[1][s].u = filled ? *(const uint4*)(kr1 + 32 * s + 8 * j) : make_uint4(0, 0, 0, 0);
    }
  };
  // ... and of its values: stored in blocks of 8 keys, [slot / 8][dim][slot % 8], so the lane's 8 keys of one
  // dimension are 16 contiguous bytes and 16 lanes read 256 contiguous bytes
  auto issue_values = [&](Frag8 (&VF)[D_TILES], int kt) {
    int ks0, ks1, vs, p0, p1, vp;
    locate(kt, p0, ks0, p1, ks1, vp, vs);
    const bf16_t* vrow = vbase + (size_t)vp * 2 * plane + ((size_t)(vs >> 3) * HEAD_DIM + n) * 8;
#pragma unroll
    for (int dt = 0; dt < D_TILES; ++dt) VF[dt].w = __builtin_nontemporal_load((const u32x4*)(vrow + dt * 16 * 8));
  };

  // S^T = K Q^T for the 32 keys of a tile
  auto scores = [&](Frag8 (&KF)[2][K32_STEPS], float4v (&st)[2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      float4v s_acc = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < K32_STEPS; ++s) s_acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(KF[t][s].v, qf[s].v, s_acc, 0, 0, 0);
      st[t] = s_acc;
    }
  };
  // masks, softmax and the value product of the tile from `kt` on
  auto finish = [&](float4v (&st)[2], Frag8 (&VF)[D_TILES], int kt) {
    const bool need_mask = kt < lo_all || kt + 31 > hi_all;
    // ---- values outside the span that any row reads are zeroed ---------------------------------- //
    const int vkey = kt + 8 * j;
    const bool boundary = (kt < lo_any) || (kt + 31 > hi_any);
    if (boundary) {
      uint32_t keep[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = vkey + e;
        if (key < lo_any || key > hi_any) keep[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
      }
#pragma unroll
      for (int dt = 0; dt < D_TILES; ++dt) {
        VF[dt].u.x &= keep[0];
        VF[dt].u.y &= keep[1];
        VF[dt].u.z &= keep[2];
        VF[dt].u.w &= keep[3];
      }
    }
    // ---- mask, running maximum, probabilities --------------------------------------------------- //
    float alpha;
    Frag8 pf;
    SOFTMAX_TILE(false, st[0], st[1], need_mask, row_valid && key >= row_start && key <= row_end && key >= key_begin && key < key_end,
                 m_run, neg_mc_run, l_run, alpha, pf)
    if (__any(alpha != 1.0f)) {  // seldom after the first tiles
      asm volatile("" ::: "memory");  // keeps this a branch: unconditional, it is 4 multiplications per output tile
#pragma unroll
      for (int dt = 0; dt < D_TILES; ++dt) acc[dt] *= alpha;
    }
    // ---- O^T += V^T P^T ------------------------------------------------------------------------- //
#pragma unroll
    for (int dt = 0; dt < D_TILES; ++dt) acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(VF[dt].v, pf.v, acc[dt], 0, 0, 0);
  };

  // wavefront w starts at the item's tile w and goes on in steps of TEAM tiles
  const int kt_step = 32 * TEAM;
  const int kt_first = (key_begin & ~31) + 32 * wave;
  Frag8 kf[2][K32_STEPS], vf[D_TILES];
  if (kt_first < key_end) {
    issue_keys(kf, kt_first);
    int kt = kt_first;
    for (; kt + kt_step < key_end; kt += kt_step) {
      float4v st[2];
      issue_values(vf, kt);
      scores(kf, st);
      issue_keys(kf, kt + kt_step);  // the next tile's keys: in flight during the softmax and the value product
      finish(st, vf, kt);
    }
    float4v st[2];
    issue_values(vf, kt);
    scores(kf, st);
    finish(st, vf, kt);
  }

  // ---- the team's wavefronts combine: the largest reference maximum, every wavefront's sums and output
  // scaled to it, and each wavefront adds up and stores a share of the dimensions ------------------------ //
  __shared__ float team_m[TEAM][16], team_l[TEAM][16];
  __shared__ __attribute__((aligned(16))) float team_o[TEAM][16][HEAD_DIM + 4];
  float l_row = l_run;
  l_row += __shfl_xor(l_row, 16, 64);
  l_row += __shfl_xor(l_row, 32, 64);
  if (j == 0) {
    team_m[wave][n] = m_run;
    team_l[wave][n] = l_row;
  }
  __syncthreads();
  float m_all = neg_inf;
#pragma unroll
  for (int w2 = 0; w2 < TEAM; ++w2) m_all = fmaxf(m_all, team_m[w2][n]);
  float l_all = 0.f, mine = 0.f;
#pragma unroll
  for (int w2 = 0; w2 < TEAM; ++w2) {
    const float mw = team_m[w2][n];  // -inf: that wavefront had no tile, or none with a key of this row
    const float f = (mw == neg_inf) ? 0.f : __builtin_amdgcn_exp2f((mw - m_all) * scale_log2e);
    l_all += team_l[w2][n] * f;
    if (w2 == wave) mine = f;
  }
#pragma unroll
  for (int dt = 0; dt < D_TILES; ++dt) *(float4v*)&team_o[wave][n][16 * dt + 4 * j] = acc[dt] * mine;
  __syncthreads();
  if (!row_valid) return;
  const float inv = page_missing ? not_a_number() : 1.0f / l_all;
  bf16_t* orow = out + (size_t)(q0 + ti) * out_stride + (size_t)hq * HEAD_DIM;
  float* prow = slot < 0 ? nullptr : partial + (((size_t)slot * n_kv_heads + g) * 16 + n) * PARTIAL_STRIDE;
  for (int dt = wave; dt < D_TILES; dt += TEAM) {
    float4v sum = *(const float4v*)&team_o[0][n][16 * dt + 4 * j];
#pragma unroll
    for (int w2 = 1; w2 < TEAM; ++w2) sum += *(const float4v*)&team_o[w2][n][16 * dt + 4 * j];
    if (slot < 0) {
      // the whole key range was this block's: normalise and store
      uint2 v;
      v.x = pack_bf16(sum[0] * inv, sum[1] * inv);
      v.y = pack_bf16(sum[2] * inv, sum[3] * inv);
      *(uint2*)(orow + 16 * dt + 4 * j) = v;
    } else {
      *(float4v*)(prow + 16 * dt + 4 * j) = sum;
    }
  }
  if (slot >= 0 && wave == 0 && j == 0) {
    prow[HEAD_DIM] = m_all * scale_log2e;  // the merge works in the scaled (log2) domain
    prow[HEAD_DIM + 1] = page_missing ? not_a_number() : l_all;  // the merged row becomes NaN too
  }
}
#undef TEAM

// ---- prompt portions: 64 * LDS_RT rows per block, keys and values shared through LDS ------- //
// work item: {sequence, first row, first key, end key (exclusive), partial slot or -1, chunks of
// the item}; one block per (item, key/value head); an item whose keys cross multiples of 8,192 is
// cut there into several such blocks, which leave partial results for the merge kernel; wavefront w takes the LDS_RT tiles of 16 rows from first_row +
// 16 * LDS_RT * w, and every operand it reads from LDS serves all of them.  Every 32-key tile of
// keys and values is fetched once per block into LDS (two buffers) and read from there as
// matrix-core operands:
//   keys   [tile t][row m][HEAD_DIM + 8]: row m of 16-key tile t is key 8*(m/4) + 4*t + m%4, so
//          the 16 lanes of one read take 16 consecutive padded rows (no bank conflicts);
//   values [8-key block][dim][8]: as in the cache, 16 lanes read 256 contiguous bytes.
// Keys outside the block's span of keys are stored as zeros, so nothing stale is multiplied.
#ifndef LDS_RT
#define LDS_RT 2  // 16-row tiles per wavefront: a block takes 64 * LDS_RT rows
#endif
#define LDS_K_STRIDE (HEAD_DIM + 8)
#define LDS_K_CHUNKS (32 * HEAD_DIM / 8)
#define LDS_V_CHUNKS (4 * HEAD_DIM)
#define LDS_K_PER_THREAD ((LDS_K_CHUNKS + 255) / 256)
#define LDS_V_PER_THREAD ((LDS_V_CHUNKS + 255) / 256)

// How a block's tiles of 32 keys reach LDS:
// LDS_STAGED (pages of a multiple of 32 keys, head sizes of a multiple of 64): every thread's share
// of a tile lies in one page, whose number is read a tile earlier; the loads are unconditional (what
// lies outside the block's span of keys is zeroed when the tile is written to LDS) and two tiles
// are in flight in registers, so that the wavefront counts its loads and waits only for the older
// tile.
// LDS_DMA (the same, head sizes 64 and 128): the loads write LDS themselves
// (global_load_lds_dwordx4: lane l of a wavefront fills bytes 16 l .. 16 l + 15 after a uniform
// address), DMA_BUFFERS - 1 tiles ahead into DMA_BUFFERS buffers, so a tile costs no registers, no
// LDS write instructions and one barrier.  Built twice: four buffers and two blocks a compute unit,
// which finishes a launch of few, uneven blocks soonest, and three buffers with at most 168
// registers for three blocks a compute unit, which hides more latency when there are many blocks.
// The rows of keys are not padded; the 16-byte piece p of row r lies at piece p ^ r (p ^ (r / 2)
// when a row has 8 pieces), which spreads the 16 rows of one matrix-core read over all banks.  Only a span's first and last tiles need zeros written over
// the values that lie outside it.  The loads and their waits are inline assembly: the compiler
// would wait for every load in flight before each LDS read.
// LDS_PLAIN: each key's page is looked up when it is fetched and one tile is in flight.
#define LDS_PLAIN 0
#define LDS_STAGED 1
#define LDS_DMA 2
// blocks a compute unit of the builds without direct loads: the accumulators of a head size above 128
// do not fit 256 registers beside the rest, so such a block has its SIMDs to itself (512 registers)
#define LDS_BLOCKS_A_UNIT (HEAD_DIM > 128 ? 1 : 2)
#define DMA_K_BYTES (32 * HEAD_DIM * 2)
#define DMA_TILE_BYTES (2 * DMA_K_BYTES)
#define DMA_HEAD_DIM_OK (HEAD_DIM == 64 || HEAD_DIM == 128)

// MIN_BLOCKS blocks share a compute unit.  With two (at most 256 registers a wavefront) or three
// (168) the compiler keeps the matrix-core accumulators in ordinary vector registers; from the
// accumulation registers every rescaling would cost a copy out and a copy back.
template <int MODE, int DMA_BUFFERS, int MIN_BLOCKS>
__global__ void __launch_bounds__(256, MIN_BLOCKS)
attention_lds_kernel(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long out_stride,
                     const bf16_t* __restrict__ cache, const int* __restrict__ block_table, int table_width,
                     const int* __restrict__ cu_q, const int* __restrict__ kv_len, const int* __restrict__ work,
                     float* __restrict__ partial, int n_kv_heads_grid, int n_q_heads, int n_kv_heads, int page_size,
                     int page_shift, int num_pages, int window_left, float scale_log2e) {
  constexpr bool FAST = MODE != LDS_PLAIN;
  constexpr int DMA_AHEAD = DMA_BUFFERS - 1;
  __shared__ __attribute__((aligned(16))) bf16_t lds_k[MODE == LDS_DMA ? 1 : 2][MODE == LDS_DMA ? 8 : 32 * LDS_K_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t lds_v[MODE == LDS_DMA ? 1 : 2][MODE == LDS_DMA ? 8 : 32 * HEAD_DIM];
  __shared__ __attribute__((aligned(16))) bf16_t lds_dma[MODE == LDS_DMA ? DMA_BUFFERS * DMA_TILE_BYTES / 2 : 8];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // the key/value head changes fastest with the block's number: workgroups go to the chip's eight XCDs in turn,
  // so with eight (or four, two) key/value heads the blocks of one head run on the same XCD(s) and find the keys
  // and values that the head's other blocks fetched in that XCD's L2
  const int item = blockIdx.x / n_kv_heads_grid;
  const int g = blockIdx.x - item * n_kv_heads_grid;
  const int* w = work + (size_t)item * WORK_INTS;
  const int b = w[0];
  const int key_begin = w[2];
  const int key_end = w[3];

  const int group = n_q_heads / n_kv_heads;
  const int q0 = cu_q[b];
  const int n_new = cu_q[b + 1] - q0;
  const int n_old = kv_len[b] - n_new;
  const int n_rows = n_new * group;

  const int n = lane & 15;
  const int j = lane >> 4;
  // this wavefront's LDS_RT tiles of 16 rows; every key and value it reads from LDS serves all of them
  bool row_valid[LDS_RT];
  int ti[LDS_RT], hq[LDS_RT], row_end[LDS_RT], row_start[LDS_RT];
  Frag8 qf[LDS_RT][K32_STEPS];
  float4v acc[LDS_RT][D_TILES];
  float m_run[LDS_RT], neg_mc_run[LDS_RT], l_run[LDS_RT];
  const float neg_inf = -__builtin_inff();
  const float lazy_raw = 8.0f / scale_log2e;  // 8 binary orders, in units of the raw scores
#pragma unroll
  for (int rt = 0; rt < LDS_RT; ++rt) {
    const int r = w[1] + 16 * (LDS_RT * wave + rt) + n;
    row_valid[rt] = r < n_rows;
    ti[rt] = row_valid[rt] ? r / group : 0;
    hq[rt] = g * group + (row_valid[rt] ? r - ti[rt] * group : 0);
    row_end[rt] = n_old + ti[rt];
    row_start[rt] = window_left >= 0 ? max(0, row_end[rt] - window_left) : 0;
    const bf16_t* qrow = q + (size_t)(q0 + ti[rt]) * q_stride + (size_t)hq[rt] * HEAD_DIM;
#pragma unroll
    for (int s = 0; s < K32_STEPS; ++s) {
      const bool filled = !(HALF_LAST_STEP && s == K32_STEPS - 1) || j < 2;
      if (row_valid[rt] && filled)
        qf[rt][s].u = *(const uint4*)(qrow + 32 * s + 8 * j);
      else
        qf[rt][s].u = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int dt = 0; dt < D_TILES; ++dt) acc[rt][dt] = (float4v){0.f, 0.f, 0.f, 0.f};
    m_run[rt] = neg_inf;
    neg_mc_run[rt] = 0.f;
    l_run[rt] = 0.f;
  }

  const size_t plane = (size_t)n_kv_heads * page_size * HEAD_DIM;
  const int* table = block_table + (size_t)b * table_width;
  const bf16_t* kbase = cache + (size_t)g * page_size * HEAD_DIM;
  const bf16_t* vbase = cache + plane + (size_t)g * page_size * HEAD_DIM;
  auto page_of = [&](int key, int& slot_in_page) -> int {
    const int lp = page_shift >= 0 ? (key >> page_shift) : (key / page_size);
    slot_in_page = key - lp * page_size;
    int page = (key >= 0 && key < key_end && lp < table_width) ? table[lp] : 0;
    return (page >= 0 && page < num_pages) ? page : 0;
  };
  // FAST: the page of the tile that starts at key kt (the same for the whole block); page 0, whose
  // contents are then zeroed, for a tile past the span of keys
  auto tile_page = [&](int kt) -> int {
    const int lp = page_shift >= 0 ? (kt >> page_shift) : (kt / page_size);
    int page = (kt < key_end && lp < table_width) ? table[lp] : 0;
    return (page >= 0 && page < num_pages) ? page : 0;
  };

  // a thread's share of one tile in registers: fetched from the cache, later written to LDS
  struct Staged {
    uint4 k[LDS_K_PER_THREAD], v[LDS_V_PER_THREAD];
  };
  auto fetch = [&](Staged& st, int kt, int page) {
    if constexpr (FAST) {
      const int lp = page_shift >= 0 ? (kt >> page_shift) : (kt / page_size);
      const int slot0 = kt - lp * page_size;  // the tile's first slot in its page
      const bf16_t* kpage = kbase + (size_t)page * 2 * plane;
      const bf16_t* vpage = vbase + (size_t)page * 2 * plane;
#pragma unroll
      for (int i = 0; i < LDS_K_PER_THREAD; ++i) {
        const int c = tid + 256 * i;
        st.k[i] = *(const uint4*)(kpage + (size_t)(slot0 + c / (HEAD_DIM / 8)) * HEAD_DIM + 8 * (c % (HEAD_DIM / 8)));
      }
#pragma unroll
      for (int i = 0; i < LDS_V_PER_THREAD; ++i) {
        const int c = tid + 256 * i;
        const int kb = c / HEAD_DIM;
        st.v[i] = *(const uint4*)(vpage + ((size_t)((slot0 >> 3) + kb) * HEAD_DIM + (c - kb * HEAD_DIM)) * 8);
      }
    } else {
#pragma unroll
      for (int i = 0; i < LDS_K_PER_THREAD; ++i) {
        const int c = tid + 256 * i;
        st.k[i] = make_uint4(0, 0, 0, 0);
        if (c < LDS_K_CHUNKS) {
          const int key = kt + c / (HEAD_DIM / 8);
          const int dp = c % (HEAD_DIM / 8);
          if (key >= key_begin && key < key_end) {
            int ks;
            const int pg = page_of(key, ks);
            st.k[i] = *(const uint4*)(kbase + (size_t)pg * 2 * plane + (size_t)ks * HEAD_DIM + 8 * dp);
          }
        }
      }
#pragma unroll
      for (int i = 0; i < LDS_V_PER_THREAD; ++i) {
        const int c = tid + 256 * i;
        st.v[i] = make_uint4(0, 0, 0, 0);
        if (c < LDS_V_CHUNKS) {
          const int kb = c / HEAD_DIM;
          const int d = c - kb * HEAD_DIM;
          const int key = kt + 8 * kb;
          if (key + 7 >= key_begin && key < key_end) {
            int vs;
            const int pg = page_of(key, vs);
            st.v[i] = *(const uint4*)(vbase + (size_t)pg * 2 * plane + ((size_t)(vs >> 3) * HEAD_DIM + d) * 8);
          }
        }
      }
    }
  };
  // writes a fetched tile to LDS, with zeros for the keys outside the block's span
  auto stash = [&](const Staged& st, int kt, int buf) {
    const bool whole = kt >= key_begin && kt + 32 <= key_end;  // all but a span's first and last tiles
    if (FAST && whole) {  // nothing to zero: the registers go to LDS as they are
#pragma unroll
      for (int i = 0; i < LDS_K_PER_THREAD; ++i) {
        const int c = tid + 256 * i;
        const int kk = c / (HEAD_DIM / 8);
        const int dp = c % (HEAD_DIM / 8);
        *(uint4*)(&lds_k[buf][(((kk >> 2) & 1) * 16 + 4 * (kk >> 3) + (kk & 3)) * LDS_K_STRIDE + 8 * dp]) = st.k[i];
      }
#pragma unroll
      for (int i = 0; i < LDS_V_PER_THREAD; ++i) *(uint4*)(&lds_v[buf][(size_t)(tid + 256 * i) * 8]) = st.v[i];
      return;
    }
#pragma unroll
    for (int i = 0; i < LDS_K_PER_THREAD; ++i) {
      const int c = tid + 256 * i;
      if (c < LDS_K_CHUNKS) {
        const int kk = c / (HEAD_DIM / 8);  // key within the tile
        const int dp = c % (HEAD_DIM / 8);
        const int t = (kk >> 2) & 1;
        const int m = 4 * (kk >> 3) + (kk & 3);
        const int key = kt + kk;
        const bool inside = whole || (key >= key_begin && key < key_end);
        *(uint4*)(&lds_k[buf][(t * 16 + m) * LDS_K_STRIDE + 8 * dp]) = inside ? st.k[i] : make_uint4(0, 0, 0, 0);
      }
    }
#pragma unroll
    for (int i = 0; i < LDS_V_PER_THREAD; ++i) {
      const int c = tid + 256 * i;
      if (c < LDS_V_CHUNKS) {
        const int key = kt + 8 * (c / HEAD_DIM);
        uint4 v = st.v[i];
        if (whole) {
        } else if (key + 7 < key_begin || key >= key_end) {
          v = make_uint4(0, 0, 0, 0);
        } else if (key < key_begin || key + 7 >= key_end) {  // the span's first or last keys: zero what lies outside
          uint32_t keep[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (key + e < key_begin || key + e >= key_end) keep[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
          v.x &= keep[0];
          v.y &= keep[1];
          v.z &= keep[2];
          v.w &= keep[3];
        }
        *(uint4*)(&lds_v[buf][(size_t)c * 8]) = v;
      }
    }
  };

  // the span of keys that any row of this wavefront reads, and the span that all of them read
  int lo_w = 0x7fffffff, hi_w = -1, lo_all = 0x7fffffff, hi_all = -1;
#pragma unroll
  for (int rt = 0; rt < LDS_RT; ++rt) {
    int lo = row_valid[rt] ? row_start[rt] : 0x7fffffff;
    int hi = row_valid[rt] ? row_end[rt] : -1;
    int lo_a = lo, hi_a = hi;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      lo = min(lo, __shfl_xor(lo, off, 64));
      hi = max(hi, __shfl_xor(hi, off, 64));
      lo_a = max(lo_a, __shfl_xor(lo_a, off, 64));
      hi_a = min(hi_a, __shfl_xor(hi_a, off, 64));
    }
    lo_w = min(lo_w, lo);
    hi_w = max(hi_w, hi);
    lo_all = rt == 0 ? lo_a : max(lo_all, lo_a);
    hi_all = rt == 0 ? hi_a : min(hi_all, hi_a);
  }

  // a key that a row of this wavefront reads must have a page, or the wavefront's rows become NaN
  const bool page_missing =
      span_lacks_page(table, table_width, num_pages, page_size, page_shift, max(lo_w, key_begin), min(hi_w, key_end - 1), lane);

  // one 32-key tile from LDS buffer `buf`: scores, running softmax, weighted values
  auto compute = [&](int kt, const bf16_t* kbuf, const bf16_t* vbuf) {
    // a wavefront whose rows all end before this tile, or start after it, has nothing to add
    if (!(kt <= hi_w && kt + 31 >= lo_w)) return;
    // ---- S^T = K Q^T ------------------------------------------------------------------ //
    float4v st[LDS_RT][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int rt = 0; rt < LDS_RT; ++rt) st[rt][t] = (float4v){0.f, 0.f, 0.f, 0.f};
      const bf16_t* krow = kbuf + (t * 16 + n) * (MODE == LDS_DMA ? HEAD_DIM : LDS_K_STRIDE);
#pragma unroll
      for (int s = 0; s < K32_STEPS; ++s) {
        const bool filled = !(HALF_LAST_STEP && s == K32_STEPS - 1) || j < 2;
        Frag8 kf;
        if constexpr (MODE == LDS_DMA)
          kf.u = *(const uint4*)(krow + 8 * ((4 * s + j) ^ (HEAD_DIM >= 128 ? n : n >> 1)));
        else
          kf.u = filled ? *(const uint4*)(krow + 8 * j + 32 * s) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int rt = 0; rt < LDS_RT; ++rt)
          st[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[rt][s].v, st[rt][t], 0, 0, 0);
      }
    }
    // ---- mask, running maximum, probabilities ------------------------------------------------ //
    const bool need_mask = kt < lo_all || kt + 31 > hi_all;
    float alpha[LDS_RT];
    Frag8 pf[LDS_RT];
    bool moved = false;
#pragma unroll
    for (int rt = 0; rt < LDS_RT; ++rt) {
      SOFTMAX_TILE(true, st[rt][0], st[rt][1], need_mask, row_valid[rt] && key >= row_start[rt] && key <= row_end[rt], m_run[rt],
                   neg_mc_run[rt], l_run[rt], alpha[rt], pf[rt])
      moved = moved || alpha[rt] != 1.0f;
    }
    if (__any(moved)) {  // seldom after the first tiles
      asm volatile("" ::: "memory");  // keeps this a branch: unconditional, it is 4 multiplications per output tile
#pragma unroll
      for (int rt = 0; rt < LDS_RT; ++rt)
#pragma unroll
        for (int dt = 0; dt < D_TILES; ++dt) {
          acc[rt][dt][0] *= alpha[rt];
          acc[rt][dt][1] *= alpha[rt];
          acc[rt][dt][2] *= alpha[rt];
          acc[rt][dt][3] *= alpha[rt];
        }
    }
    // ---- O^T += V^T P^T ------------------------------------------------------------------- //
    const bf16_t* vrow = vbuf + ((size_t)j * HEAD_DIM + n) * 8;
#pragma unroll
    for (int dt = 0; dt < D_TILES; ++dt) {
      Frag8 vf;
      vf.u = *(const uint4*)(vrow + dt * 16 * 8);
#pragma unroll
      for (int rt = 0; rt < LDS_RT; ++rt) {
        acc[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[rt].v, acc[rt][dt], 0, 0, 0);
      }
    }
  };

  const int kt_first = key_begin & ~31;
  const int n_tiles = (key_end - kt_first + 31) / 32;
  if constexpr (MODE == LDS_DMA) {
    // tile t lies in buffer t % DMA_BUFFERS; its loads are issued DMA_AHEAD tiles ahead, after the
    // barrier that ends the use of that buffer by tile t - 1
    // the queries arrive before the first of these loads: the compiler, which does not see them,
    // would otherwise wait for "everything" at the queries' first use inside the loop
#pragma unroll
    for (int rt = 0; rt < LDS_RT; ++rt)
#pragma unroll
      for (int s = 0; s < K32_STEPS; ++s)
        asm volatile("" : : "v"(qf[rt][s].u.x), "v"(qf[rt][s].u.y), "v"(qf[rt][s].u.z), "v"(qf[rt][s].u.w));
    const uint32_t lds0 = (uint32_t)(uintptr_t)(&lds_dma[0]);
    // loads per thread and tile (at least 1 so that the code also parses for head sizes that never run it)
    constexpr int KPT = MODE == LDS_DMA && LDS_K_CHUNKS >= 256 ? LDS_K_CHUNKS / 256 : 1;
    constexpr int VPT = MODE == LDS_DMA && LDS_V_CHUNKS >= 256 ? LDS_V_CHUNKS / 256 : 1;
    constexpr int CH = HEAD_DIM / 8;                                    // 16-byte pieces in a row of keys
    uint32_t k_off[KPT], v_off[VPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int c = (4 * i + wave) * 64 + lane;  // the piece of LDS that this lane fills
      const int r = c / CH;                      // row: tile t = r / 16, row m = r % 16 of it
      const int m = r & 15;
      const int kk = ((m >> 2) << 3) | ((r >> 4) << 2) | (m & 3);
      const int dp = (c % CH) ^ (HEAD_DIM >= 128 ? m : m >> 1);
      k_off[i] = (uint32_t)(kk * HEAD_DIM + 8 * dp) * 2;
    }
    // a tile's values lie `plane` elements after its keys, at the same offset within the page
#pragma unroll
    for (int i = 0; i < VPT; ++i) v_off[i] = (uint32_t)(plane * 2) + (uint32_t)((4 * i + wave) * 64 + lane) * 16;
    // where the next tile to be loaded lies: its first key, its slot in its page, that page's keys
    // in the cache, and the table's entry for the page after it, read a page ahead; all uniform
    int issue_kt = kt_first;
    int issue_lp = page_shift >= 0 ? (kt_first >> page_shift) : (kt_first / page_size);
    int issue_slot = kt_first - issue_lp * page_size;
    auto entry = [&](int lp) -> int { return lp < table_width ? table[lp] : 0; };
    auto page_keys = [&](int raw, int kt) -> const bf16_t* {
      const int page = (kt < key_end && raw >= 0 && raw < num_pages) ? raw : 0;  // past the span: any page, never used
      return kbase + (size_t)page * 2 * plane;
    };
    const bf16_t* issue_page = page_keys(entry(issue_lp), issue_kt);
    int entry_after = entry(issue_lp + 1);
    auto dma_next_tile = [&](int b) {
      const bf16_t* src = issue_page + (size_t)issue_slot * HEAD_DIM;
      const uint32_t dst = lds0 + b * DMA_TILE_BYTES + wave * 1024;
#pragma unroll
      for (int i = 0; i < KPT; ++i) dma16(src, k_off[i], dst + i * 4096);
#pragma unroll
      for (int i = 0; i < VPT; ++i) dma16(src, v_off[i], dst + DMA_K_BYTES + i * 4096);
      issue_kt += 32;
      issue_slot += 32;
      if (issue_slot == page_size) {
        issue_slot = 0;
        ++issue_lp;
        issue_page = page_keys(entry_after, issue_kt);
        entry_after = entry(issue_lp + 1);
      }
    };
    // zeros over the values of keys outside the block's span (their scores are masked, but what
    // lies there may be anything, also not a number)
    auto zero_outside = [&](int kt, bf16_t* vbuf) {
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int c = tid + 256 * i;
        const int key = kt + 8 * (c / HEAD_DIM);
        if (key >= key_begin && key + 8 <= key_end) continue;
        uint4 v = *(uint4*)(vbuf + (size_t)c * 8);
        uint32_t keep[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (key + e < key_begin || key + e >= key_end) keep[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
        v.x &= keep[0];
        v.y &= keep[1];
        v.z &= keep[2];
        v.w &= keep[3];
        *(uint4*)(vbuf + (size_t)c * 8) = v;
      }
    };
#pragma unroll
    for (int t = 0; t < DMA_AHEAD; ++t) dma_next_tile(t);
    for (int it = 0; it < n_tiles; it += DMA_BUFFERS) {
#pragma unroll
      for (int u = 0; u < DMA_BUFFERS; ++u) {
        const int kt = kt_first + 32 * (it + u);
        // this thread's loads of tile it + u have landed (those of the tiles after it may be in flight);
        // after the barrier so have everyone's, and everyone has left tile it + u - 1
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"((DMA_AHEAD - 1) * (KPT + VPT)) : "memory");
        dma_next_tile((u + DMA_AHEAD) % DMA_BUFFERS);
        if (it + u < n_tiles) {
          bf16_t* kbuf = lds_dma + u * (DMA_TILE_BYTES / 2);
          bf16_t* vbuf = kbuf + DMA_K_BYTES / 2;
          if (kt < key_begin || kt + 32 > key_end) {  // a span's first or last tile
            zero_outside(kt, vbuf);
            __syncthreads();
          }
          compute(kt, kbuf, vbuf);
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // the loads past the last tile
  } else if constexpr (FAST) {
    // tile t waits in registers set t % 2 and is multiplied from LDS buffer t % 2; its fetch is
    // issued three tiles ahead of its use and has two iterations to arrive
    Staged sa, sb;
    fetch(sa, kt_first, tile_page(kt_first));
    fetch(sb, kt_first + 32, tile_page(kt_first + 32));
    int page_next = tile_page(kt_first + 64);
    stash(sa, kt_first, 0);
    fetch(sa, kt_first + 64, page_next);
    page_next = tile_page(kt_first + 96);
    __syncthreads();
    for (int it = 0; it < n_tiles; it += 2) {
      const int kt = kt_first + 32 * it;
      compute(kt, lds_k[0], lds_v[0]);
      stash(sb, kt + 32, 1);
      fetch(sb, kt + 96, page_next);
      page_next = tile_page(kt + 128);
      __syncthreads();
      if (it + 1 < n_tiles) compute(kt + 32, lds_k[1], lds_v[1]);
      stash(sa, kt + 64, 0);
      fetch(sa, kt + 128, page_next);
      page_next = tile_page(kt + 160);
      __syncthreads();
    }
  } else {
    Staged sa;
    fetch(sa, kt_first, 0);
    stash(sa, kt_first, 0);
    if (n_tiles > 1) fetch(sa, kt_first + 32, 0);
    __syncthreads();
    for (int it = 0; it < n_tiles; ++it) {
      const int kt = kt_first + 32 * it;
      const int buf = it & 1;
      compute(kt, lds_k[buf], lds_v[buf]);
      // tile it + 1 (fetched an iteration ago) goes into the other buffer, which every wavefront
      // left at the last barrier; then tile it + 2 is fetched
      if (it + 1 < n_tiles) stash(sa, kt + 32, buf ^ 1);
      if (it + 2 < n_tiles) fetch(sa, kt + 64, 0);
      __syncthreads();
    }
  }

#pragma unroll
  for (int rt = 0; rt < LDS_RT; ++rt) {
    float l_row = l_run[rt];
    l_row += __shfl_xor(l_row, 16, 64);
    l_row += __shfl_xor(l_row, 32, 64);
    if (!row_valid[rt]) continue;
    if (w[4] >= 0) {
      // the item's keys are cut into w[5] chunks and this block had one of them: its row tile t
      // leaves what it has at slot w[4] + t * w[5], in the form of the split kernel's partial results
      const int slot = w[4] + (LDS_RT * wave + rt) * w[5];
      float* prow = partial + (((size_t)slot * n_kv_heads + g) * 16 + n) * PARTIAL_STRIDE;
#pragma unroll
      for (int dt = 0; dt < D_TILES; ++dt) *(float4v*)(prow + 16 * dt + 4 * j) = acc[rt][dt];
      if (j == 0) {
        prow[HEAD_DIM] = m_run[rt] * scale_log2e;
        prow[HEAD_DIM + 1] = page_missing ? not_a_number() : l_row;
      }
      continue;
    }
    const float inv = page_missing ? not_a_number() : 1.0f / l_row;
    bf16_t* orow = out + (size_t)(q0 + ti[rt]) * out_stride + (size_t)hq[rt] * HEAD_DIM;
#pragma unroll
    for (int dt = 0; dt < D_TILES; ++dt) {
      uint2 v;
      v.x = pack_bf16(acc[rt][dt][0] * inv, acc[rt][dt][1] * inv);
      v.y = pack_bf16(acc[rt][dt][2] * inv, acc[rt][dt][3] * inv);
      *(uint2*)(orow + 16 * dt + 4 * j) = v;
    }
  }
}

// merge item: {sequence, first row, first partial slot, number of partials}
// One block per (item, key/value head, row): wavefront w takes partials w, w + MERGE_WAVES, ...
// (a wavefront's partials come one after the other, so more wavefronts mean a shorter chain of
// loads), the lanes of a wavefront the dimensions; the running sums are added in wavefront order.
// MERGE_WAVES: 16 for items of more than 32 partials, 4 up to 32, 1 for the few partials of the blocks
// that share keys through LDS (there the rows are many).
template <int MERGE_WAVES>
__global__ void __launch_bounds__(MERGE_WAVES * 64)
attention_merge_kernel(bf16_t* __restrict__ out, long out_stride, const float* __restrict__ partial,
                       const int* __restrict__ cu_q, const int* __restrict__ merge, int n_q_heads, int n_kv_heads) {
  __shared__ float red_max[MERGE_WAVES];
  __shared__ float red_l[MERGE_WAVES];
  __shared__ float red_o[MERGE_WAVES][HEAD_DIM];
  const int item = blockIdx.x;
  const int g = blockIdx.y;
  const int n = blockIdx.z;
  const int lane = threadIdx.x & 63;
  const int wave = MERGE_WAVES == 1 ? 0 : (int)(threadIdx.x >> 6);
  const int* mi = merge + (size_t)item * 4;
  const int b = mi[0];
  const int row0 = mi[1];
  const int first = mi[2];
  const int count = mi[3];
  const int group = n_q_heads / n_kv_heads;
  const int q0 = cu_q[b];
  const int n_rows = (cu_q[b + 1] - q0) * group;
  const int r = row0 + n;
  if (r >= n_rows) return;
  const int ti = r / group;
  const int hq = g * group + (r - ti * group);
  const float neg_inf = -__builtin_inff();
  const float* base = partial + (((size_t)first * n_kv_heads + g) * 16 + n) * PARTIAL_STRIDE;
  const size_t step = (size_t)n_kv_heads * 16 * PARTIAL_STRIDE;

  // the row's maximum over all partials
  float m_all = neg_inf;
  for (int s = threadIdx.x; s < count; s += MERGE_WAVES * 64) m_all = fmaxf(m_all, base[(size_t)s * step + HEAD_DIM]);
  m_all = wave_max(m_all);
  if (lane == 0) red_max[wave] = m_all;
  __syncthreads();
  m_all = red_max[0];
#pragma unroll
  for (int w = 1; w < MERGE_WAVES; ++w) m_all = fmaxf(m_all, red_max[w]);

  float o[(HEAD_DIM + 63) / 64];
#pragma unroll
  for (int i = 0; i < (HEAD_DIM + 63) / 64; ++i) o[i] = 0.f;
  float l_part = 0.f;
  for (int s = wave; s < count; s += MERGE_WAVES) {
    const float* prow = base + (size_t)s * step;
    const float ms = prow[HEAD_DIM];
    const float wgt = (ms == neg_inf) ? 0.f : exp2f(ms - m_all);  // -inf: the row had no key in that chunk
    l_part += prow[HEAD_DIM + 1] * wgt;
#pragma unroll
    for (int i = 0; i < (HEAD_DIM + 63) / 64; ++i) {
      const int d = lane + 64 * i;
      if (d < HEAD_DIM) o[i] += prow[d] * wgt;
    }
  }
  if (lane == 0) red_l[wave] = l_part;
#pragma unroll
  for (int i = 0; i < (HEAD_DIM + 63) / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < HEAD_DIM) red_o[wave][d] = o[i];
  }
  __syncthreads();
  if (wave != 0) return;
  float l_all = 0.f;
#pragma unroll
  for (int w = 0; w < MERGE_WAVES; ++w) l_all += red_l[w];
  const float inv = 1.0f / l_all;
  bf16_t* orow = out + (size_t)(q0 + ti) * out_stride + (size_t)hq * HEAD_DIM;
#pragma unroll
  for (int i = 0; i < (HEAD_DIM + 63) / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < HEAD_DIM) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < MERGE_WAVES; ++w) sum += red_o[w][d];
      orow[d] = f32_to_bf16(sum * inv);
    }
  }
}

extern "C" int cwm_attention_mfma(const void* q, long q_stride, void* out, long out_stride, const void* cache,
                                  const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                                  const int* work, int n_work, int work_keys, const int* work_wide, int n_work_wide, int wide_tiles,
                                  int wide_three_blocks, const int* merge,
                                  int n_merge, int n_merge_mid, int n_merge_few, float* partial, int n_q_heads, int n_kv_heads, int head_dim,
                                  int page_size, int num_pages, int window_left, float scale, hipStream_t stream) {
  // `work`: items of one 16-row tile (may be split over chunks of keys), one wavefront each;
  // `work_wide`: items of 4 * LDS_RT row tiles, one block each with keys and values in LDS
  CWM_REQUIRE(head_dim == HEAD_DIM, "attention_mfma: this library is built for head_dim %d, not %d", HEAD_DIM, head_dim);
  CWM_REQUIRE(n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0,
              "attention_mfma: %d query heads do not divide into %d key/value heads", n_q_heads, n_kv_heads);
  CWM_REQUIRE(page_size > 0 && page_size % 8 == 0, "attention_mfma: page size %d must be a multiple of 8", page_size);
  CWM_REQUIRE(num_pages > 0 && table_width > 0, "attention_mfma: bad cache geometry");
  CWM_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0, "attention_mfma: token strides must keep 16-byte alignment");
  CWM_REQUIRE(n_work >= 0 && n_work_wide >= 0 && n_merge >= 0, "attention_mfma: negative work counts");
  CWM_REQUIRE(n_work_wide == 0 || wide_tiles == 4 * LDS_RT, "attention_mfma: wide items must have %d row tiles, not %d",
              4 * LDS_RT, wide_tiles);
  CWM_REQUIRE(n_merge == 0 || partial != nullptr, "attention_mfma: partial buffer missing");
  const float scale_log2e = scale * 1.4426950408889634f;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  int status = 0;
  if (n_work > 0) {
    // a block of four wavefronts per (item, key/value head)
    const long long blocks = (long long)n_work * n_kv_heads;
    CWM_REQUIRE(blocks <= 0x7fffffffLL, "attention_mfma: too many work items");
    (void)work_keys;
#define CWM_LAUNCH_TEAM(PAGE32)                                                                                          \
  hipLaunchKernelGGL((attention_mfma_kernel<PAGE32>), dim3((unsigned)blocks), dim3(256), 0, stream, (const bf16_t*)q,     \
                     q_stride, (bf16_t*)out, out_stride, (const bf16_t*)cache, block_table, table_width, cu_q, kv_len,   \
                     work, n_work, partial, n_q_heads, n_kv_heads, page_size, page_shift, num_pages, window_left,        \
                     scale_log2e)
    if (page_size % 32 == 0)
      CWM_LAUNCH_TEAM(true);
    else
      CWM_LAUNCH_TEAM(false);
#undef CWM_LAUNCH_TEAM
    status = cwm_launch_status("attention_mfma");
    if (status) return status;
  }
  if (n_work_wide > 0) {
    const long long blocks = (long long)n_work_wide * n_kv_heads;
    CWM_REQUIRE(blocks <= 0x7fffffffLL, "attention_mfma: too many work items");
#define CWM_LAUNCH_LDS(MODE, BUFFERS, MIN_BLOCKS)                                                                        \
  hipLaunchKernelGGL((attention_lds_kernel<MODE, BUFFERS, MIN_BLOCKS>), dim3((unsigned)blocks), dim3(256), 0, stream,     \
                     (const bf16_t*)q, q_stride,                                                                          \
                     (bf16_t*)out, out_stride, (const bf16_t*)cache, block_table, table_width, cu_q, kv_len, work_wide,   \
                     partial, n_kv_heads, n_q_heads, n_kv_heads, page_size, page_shift, num_pages, window_left, scale_log2e)
    // tiles of 32 keys that never straddle a page, and shares of a tile that divide evenly over the block
    if (page_size % 32 == 0 && LDS_K_CHUNKS % 256 == 0 && LDS_V_CHUNKS % 256 == 0) {
#if DMA_HEAD_DIM_OK
      // the values' offset from the keys of a page must fit the loads' 32-bit offsets
      if ((unsigned long long)n_kv_heads * page_size * HEAD_DIM * 2 >= (1ull << 31))
        CWM_LAUNCH_LDS(LDS_STAGED, 2, LDS_BLOCKS_A_UNIT);
      else if (wide_three_blocks)  // the caller's choice: three blocks a compute unit
        CWM_LAUNCH_LDS(LDS_DMA, 3, 3);
      else
        CWM_LAUNCH_LDS(LDS_DMA, 4, 2);
#else
      CWM_LAUNCH_LDS(LDS_STAGED, 2, LDS_BLOCKS_A_UNIT);
#endif
    } else {
      CWM_LAUNCH_LDS(LDS_PLAIN, 2, LDS_BLOCKS_A_UNIT);
    }
#undef CWM_LAUNCH_LDS
    status = cwm_launch_status("attention_lds");
    if (status) return status;
  }
  if (n_merge > 0) {
    CWM_REQUIRE(n_kv_heads <= 65535, "attention_mfma: too many key/value heads for the merge grid");
    // the list holds the items with many partials, then n_merge_mid items with at most 32, then n_merge_few
    // items of blocks of many rows whose keys were cut (few partials each)
    CWM_REQUIRE(n_merge_few >= 0 && n_merge_mid >= 0 && n_merge_few + n_merge_mid <= n_merge, "attention_mfma: bad counts of merge items");
    const int n_many = n_merge - n_merge_mid - n_merge_few;
#define CWM_LAUNCH_MERGE(WAVES, COUNT, FIRST)                                                                              \
  if ((COUNT) > 0)                                                                                                        \
  hipLaunchKernelGGL(attention_merge_kernel<WAVES>, dim3(COUNT, n_kv_heads, 16), dim3(WAVES * 64), 0, stream, (bf16_t*)out, \
                     out_stride, (const float*)partial, cu_q, merge + (size_t)(FIRST) * 4, n_q_heads, n_kv_heads)
    CWM_LAUNCH_MERGE(16, n_many, 0);
    CWM_LAUNCH_MERGE(4, n_merge_mid, n_many);
    CWM_LAUNCH_MERGE(1, n_merge_few, n_many + n_merge_mid);
#undef CWM_LAUNCH_MERGE
    status = cwm_launch_status("attention_merge");
  }
  return status;
}
