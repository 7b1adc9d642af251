// Next-token choice from float32 logits, one block per row: greedy argmax, or a
// draw from softmax(logits / T) restricted to the nucleus of mass top_p.
//
// Reference semantics: argmax when sampling is off (cwm/fastgen/generate.py:1012);
// probs = softmax(logits / T) in float32 (:1003); nucleus = the entries whose
// preceding mass in descending order does not exceed top_p, renormalised
// (cwm/fastgen/utils/sampling.py:38-45).  The draw itself uses a uniform number
// u in [0, 1) that the caller supplies per row: the first kept entry, in vocabulary
// order, at which the running kept mass exceeds u * (kept mass).  That is a draw
// from the same distribution as torch.multinomial, made reproducible per request.
//
// Also returned per row: logprob = log softmax(logits)[token] (the reference's
// -cross_entropy, generate.py:1010) and sample_logprob = log of the probability
// under the temperature / nucleus distribution (0 for greedy rows).
//
// The nucleus is found without sorting: with e_i = exp((x_i - max) / T) and
// f(t) = sum of e_i > t, the kept set is {e_i >= t*} for the smallest float t*
// with f(t*) <= top_p * sum(e); t* is found by cutting the interval of bit patterns.
// Entries exactly equal to the threshold are all kept.  Without a nucleus (top_p = 1)
// nothing is stored: the draw recomputes e_i where it walks.  A row of 128k logits
// takes about 22 us greedy, 44 us at a temperature and 170 us with a nucleus.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

CWM_DEFINE_ERROR_API

#define SAMPLE_THREADS 1024

struct MaxIdx {
  float v;
  int i;
};

__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

// f(i, x[i]) for every i < n, thread t taking i = t, t + THREADS, ... in increasing order; VEC (n a multiple of 4
// and x 16-byte aligned): four adjacent entries at a time, so a pass over a row of 128k logits is 32 loads a thread
template <bool VEC, typename F>
__device__ __forceinline__ void each_strided(const float* x, int n, int tid, F&& f) {
  if (VEC) {
    const float4* x4 = (const float4*)x;
#pragma unroll 2
    for (int i = tid; i < (n >> 2); i += SAMPLE_THREADS) {
      const float4 v = x4[i];
      f(4 * i, v.x);
      f(4 * i + 1, v.y);
      f(4 * i + 2, v.z);
      f(4 * i + 3, v.w);
    }
  } else {
#pragma unroll 4
    for (int i = tid; i < n; i += SAMPLE_THREADS) f(i, x[i]);
  }
}

#ifndef SEARCH_WAYS
#define SEARCH_WAYS 2  // thresholds tried in one pass over the row (measured at 128k entries: 2 169 us, 3 187, 4 196, 8 242)
#endif

template <bool VEC>
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, long row_stride, int vocab, const float* __restrict__ temperature,
              const float* __restrict__ top_p, const float* __restrict__ uniform, float* __restrict__ workspace,
              int* __restrict__ token_out, float* __restrict__ logprob_out, float* __restrict__ sample_logprob_out) {
  __shared__ float scratch[16];
  __shared__ float mv[SAMPLE_THREADS / CWM_WAVE];
  __shared__ int mi[SAMPLE_THREADS / CWM_WAVE];
  __shared__ float seg_sum[2 * SAMPLE_THREADS / CWM_WAVE];  // masses of the 16 regions, then of the chosen region's 16 parts
  __shared__ float above_part[SAMPLE_THREADS / CWM_WAVE][SEARCH_WAYS];

  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float* x = logits + (size_t)row * row_stride;
  float* e = workspace + (size_t)row * vocab;

  // 1. maximum and its first index
  MaxIdx best = {-__builtin_inff(), 0x7fffffff};
  each_strided<VEC>(x, vocab, tid, [&](int i, float v) {
    if (v > best.v) {  // a thread visits its indices in increasing order
      best.v = v;
      best.i = i;
    }
  });
#pragma unroll
  for (int off = CWM_WAVE / 2; off > 0; off >>= 1) {
    MaxIdx o;
    o.v = __shfl_xor(best.v, off, CWM_WAVE);
    o.i = __shfl_xor(best.i, off, CWM_WAVE);
    best = better(best, o);
  }
  if ((tid & (CWM_WAVE - 1)) == 0) {
    mv[tid / CWM_WAVE] = best.v;
    mi[tid / CWM_WAVE] = best.i;
  }
  __syncthreads();
  best.v = mv[0];
  best.i = mi[0];
  for (int w = 1; w < SAMPLE_THREADS / CWM_WAVE; ++w) {
    MaxIdx o = {mv[w], mi[w]};
    best = better(best, o);
  }
  if (best.i >= vocab) best.i = 0;  // every logit NaN or -inf: still return a valid id
  const float xmax = best.v;

  // 2. log-sum-exp at temperature 1
  float s1 = 0.f;
  each_strided<VEC>(x, vocab, tid, [&](int, float v) { s1 += expf(v - xmax); });
  s1 = block_sum(s1, scratch);
  const float lse = xmax + logf(s1);

  const float temp = temperature[row];
  if (!(temp > 0.f)) {  // greedy
    if (tid == 0) {
      token_out[row] = best.i;
      logprob_out[row] = xmax - lse;
      sample_logprob_out[row] = 0.f;
    }
    return;
  }

  // 3. the nucleus threshold (top_p < 1 only): unnormalised probabilities at temperature T go to the
  //    workspace, and the search reads them from there.  f(t) = sum of e_i > t, summed in a fixed order, does
  //    not grow with t, so the smallest t with f(t) <= top_p * sum(e) is found by cutting the interval of bit
  //    patterns: SEARCH_WAYS thresholds a pass, each with a sum of its own.
  const float inv_t = 1.0f / temp;
  const float tp = top_p[row];
  const bool nucleus = tp < 1.0f;
  float thresh = 0.f;
  if (nucleus) {
    float z = 0.f;
    if (VEC) {
      float4* e4 = (float4*)e;
      const float4* x4 = (const float4*)x;
#pragma unroll 2
      for (int i = tid; i < (vocab >> 2); i += SAMPLE_THREADS) {
        const float4 v = x4[i];
        float4 ev;
        ev.x = expf((v.x - xmax) * inv_t);
        ev.y = expf((v.y - xmax) * inv_t);
        ev.z = expf((v.z - xmax) * inv_t);
        ev.w = expf((v.w - xmax) * inv_t);
        e4[i] = ev;
        z += ev.x;
        z += ev.y;
        z += ev.z;
        z += ev.w;
      }
    } else {
#pragma unroll 4
      for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
        const float ev = expf((x[i] - xmax) * inv_t);
        e[i] = ev;
        z += ev;
      }
    }
    z = block_sum(z, scratch);  // (its first barrier also orders the writes of e before the reads below)
    const float target = tp * z;
    uint32_t lo = 0u, hi = __float_as_uint(1.0f);  // f(1) = 0: the answer lies in [lo, hi]
    while (lo < hi) {
      // thresholds lo <= m_0 < m_1 < ... < hi, evenly spread (the same one several times once the interval is short)
      uint32_t m[SEARCH_WAYS];
      float above[SEARCH_WAYS];
      const uint32_t span = hi - lo;
#pragma unroll
      for (int j = 0; j < SEARCH_WAYS; ++j) {
        m[j] = lo + (uint32_t)(((unsigned long long)span * (j + 1)) / (SEARCH_WAYS + 1));
        if (m[j] >= hi) m[j] = hi - 1;
        above[j] = 0.f;
      }
      each_strided<VEC>(e, vocab, tid, [&](int, float ev) {
#pragma unroll
        for (int j = 0; j < SEARCH_WAYS; ++j) above[j] += ev > __uint_as_float(m[j]) ? ev : 0.f;
      });
#pragma unroll
      for (int j = 0; j < SEARCH_WAYS; ++j) above[j] = wave_sum(above[j]);
      __syncthreads();
      if ((tid & (CWM_WAVE - 1)) == 0) {
#pragma unroll
        for (int j = 0; j < SEARCH_WAYS; ++j) above_part[tid / CWM_WAVE][j] = above[j];
      }
      __syncthreads();
      // the first threshold whose sum is small enough becomes the upper end, the one before it (plus one) the lower
      int first = SEARCH_WAYS;
#pragma unroll
      for (int j = SEARCH_WAYS - 1; j >= 0; --j) {
        float total = 0.f;
        for (int w = 0; w < SAMPLE_THREADS / CWM_WAVE; ++w) total += above_part[w][j];
        if (total <= target) first = j;
      }
      if (first > 0) lo = m[first - 1] + 1;
      if (first < SEARCH_WAYS) hi = m[first];
    }
    thresh = __uint_as_float(hi);
  }
  // the kept mass of entry i (0 for an entry outside the nucleus); without a nucleus it is computed anew
  // wherever it is needed, which is cheaper than a trip through memory
  auto kept = [&](int i) -> float {
    const float ev = nucleus ? e[i] : expf((x[i] - xmax) * inv_t);
    return ev >= thresh ? ev : 0.f;
  };

  // 4. inverse CDF over the kept entries in vocabulary order, in three levels: the vocabulary is cut into 16
  //    regions of whole groups of 64 entries, one per wavefront, whose masses say in which region the drawn
  //    point lies; that region into 16 parts likewise; the part is then walked group by group by one wavefront.
  //    Every load is of 64 adjacent entries.  The sums of the three levels are rounded differently, so a level
  //    may find the point beyond its last mass: it then takes its last entry with mass.
  const int lane = tid & (CWM_WAVE - 1);
  const int wave = tid / CWM_WAVE;
  constexpr int WAVES = SAMPLE_THREADS / CWM_WAVE;
  const int n_groups = (vocab + CWM_WAVE - 1) / CWM_WAVE;
  // mass of the entries [begin, end) that this wavefront's lanes read side by side
  auto wave_mass = [&](int begin, int end) -> float {
    float m = 0.f;
    if (VEC) {  // begin is a multiple of 64 and end of 4
      const float4* src = (const float4*)((nucleus ? e : x) + begin);
#pragma unroll 2
      for (int i = lane; i < ((end - begin) >> 2); i += CWM_WAVE) {
        const float4 v = src[i];
        const float e0 = nucleus ? v.x : expf((v.x - xmax) * inv_t), e1 = nucleus ? v.y : expf((v.y - xmax) * inv_t);
        const float e2 = nucleus ? v.z : expf((v.z - xmax) * inv_t), e3 = nucleus ? v.w : expf((v.w - xmax) * inv_t);
        m += e0 >= thresh ? e0 : 0.f;
        m += e1 >= thresh ? e1 : 0.f;
        m += e2 >= thresh ? e2 : 0.f;
        m += e3 >= thresh ? e3 : 0.f;
      }
    } else {
#pragma unroll 4
      for (int i = begin + lane; i < end; i += CWM_WAVE) m += kept(i);
    }
    return wave_sum(m);
  };
  // the first of the WAVES masses in `part` at which the running sum from `before` passes `target` (the last
  // one with mass if none does); the running sum before it is returned through `before`
  auto pick_part = [&](const float* part, float target, float& before) -> int {
    float run = before;
    int pick = -1, last = 0;
    float pick_before = before, last_before = before;
    for (int w = 0; w < WAVES; ++w) {
      const float m = part[w];
      if (m > 0.f) {
        last = w;
        last_before = run;
        if (pick < 0 && run + m > target) {
          pick = w;
          pick_before = run;
        }
      }
      run += m;
    }
    before = pick < 0 ? last_before : pick_before;
    return pick < 0 ? last : pick;
  };

  const int region_groups = (n_groups + WAVES - 1) / WAVES;
  {
    const int begin = min(vocab, wave * region_groups * CWM_WAVE);
    const float m = wave_mass(begin, min(vocab, begin + region_groups * CWM_WAVE));
    if (lane == 0) seg_sum[wave] = m;
  }
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < WAVES; ++w) total += seg_sum[w];
  const float target = uniform[row] * total;
  float before = 0.f;
  const int region = pick_part(seg_sum, target, before);  // the same in every thread

  const int part_groups = (region_groups + WAVES - 1) / WAVES;
  const int region_begin = min(vocab, region * region_groups * CWM_WAVE);
  const int region_end = min(vocab, region_begin + region_groups * CWM_WAVE);
  {
    const int begin = min(region_end, region_begin + wave * part_groups * CWM_WAVE);
    const float m = wave_mass(begin, min(region_end, begin + part_groups * CWM_WAVE));
    if (lane == 0) seg_sum[WAVES + wave] = m;
  }
  __syncthreads();
  const int part = pick_part(seg_sum + WAVES, target, before);

  if (wave == 0) {
    const int begin = min(region_end, region_begin + part * part_groups * CWM_WAVE);
    const int end = min(region_end, begin + part_groups * CWM_WAVE);
    float run = before;
    int tok = -1;  // the entry at which the running sum passes the target
    int last_tok = -1;  // the last entry with mass so far, in case rounding puts the target beyond the part's mass
    for (int g = begin; g < end && tok < 0; g += CWM_WAVE) {
      const int i = g + lane;
      const float v = i < end ? kept(i) : 0.f;
      float scan = v;  // inclusive sum over the lanes up to this one
#pragma unroll
      for (int off = 1; off < CWM_WAVE; off <<= 1) {
        const float o = __shfl_up(scan, off, CWM_WAVE);
        if (lane >= off) scan += o;
      }
      const unsigned long long has_mass = __ballot(v > 0.f);
      const unsigned long long passes = __ballot(v > 0.f && run + scan > target);
      if (passes) tok = g + __ffsll((long long)passes) - 1;
      if (has_mass) last_tok = g + 63 - __clzll((long long)has_mass);
      run += __shfl(scan, CWM_WAVE - 1, CWM_WAVE);
    }
    if (tok < 0) tok = last_tok;
    if (lane == 0) {
      if (tok < 0) tok = best.i;  // no entry with mass at all (every logit NaN)
      token_out[row] = tok;
      logprob_out[row] = x[tok] - lse;
      sample_logprob_out[row] = logf(kept(tok) / total);
    }
  }
}

static void launch_sample(const float* logits, long row_stride, int n_rows, int vocab, const float* temperature, const float* top_p,
                          const float* uniform, float* workspace, int* token_out, float* logprob_out, float* sample_logprob_out,
                          hipStream_t stream) {
  // four entries a load where every row of the logits and of the workspace starts at a multiple of 16 bytes
  const bool vec = vocab % 4 == 0 && row_stride % 4 == 0 && (uintptr_t)logits % 16 == 0 && (uintptr_t)workspace % 16 == 0;
  if (vec)
    hipLaunchKernelGGL(sample_kernel<true>, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride, vocab, temperature,
                       top_p, uniform, workspace, token_out, logprob_out, sample_logprob_out);
  else
    hipLaunchKernelGGL(sample_kernel<false>, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride, vocab, temperature,
                       top_p, uniform, workspace, token_out, logprob_out, sample_logprob_out);
}

extern "C" int cwm_sample(const float* logits, long row_stride, int n_rows, int vocab, const float* temperature,
                          const float* top_p, const float* uniform, float* workspace, int* token_out,
                          float* logprob_out, float* sample_logprob_out, hipStream_t stream) {
  CWM_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", n_rows, vocab);
  CWM_REQUIRE(row_stride >= vocab, "sample: row stride shorter than the vocabulary");
  CWM_REQUIRE(workspace != nullptr, "sample: workspace missing");
  if (n_rows == 0) return 0;
  launch_sample(logits, row_stride, n_rows, vocab, temperature, top_p, uniform, workspace, token_out, logprob_out, sample_logprob_out, stream);
  return cwm_launch_status("sample");
}

// ---- the same without a workspace argument: nothing is allocated ------------------ //
// The unnormalised probabilities go to a device array of this file; see no_alloc.h.
// In host code `sample_scratch` is only a stand-in for the symbol: its device address
// differs from GPU to GPU and is looked up once per device, with that device current.
static __device__ __align__(256) float sample_scratch[CWM_SAMPLE_STATIC_MAX_FLOATS];

#define CWM_MAX_DEVICES 64
static float* sample_scratch_ptr[CWM_MAX_DEVICES] = {nullptr};
static std::mutex sample_scratch_mutex;

extern "C" long cwm_sample_static_capacity() { return CWM_SAMPLE_STATIC_MAX_FLOATS; }

// The array's address on the current device, looked up at the first call there.  Sets `*out`; returns non-zero on failure.
static int sample_scratch_on_current_device(float** out) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return cwm_fail("sample_static: hipGetDevice failed: %s", hipGetErrorString(err));
  CWM_REQUIRE(device >= 0 && device < CWM_MAX_DEVICES, "sample_static: device %d is outside 0..%d", device, CWM_MAX_DEVICES - 1);
  std::lock_guard<std::mutex> guard(sample_scratch_mutex);
  if (sample_scratch_ptr[device] == nullptr) {
    void* found = nullptr;
    err = hipGetSymbolAddress(&found, HIP_SYMBOL(sample_scratch));
    if (err != hipSuccess || found == nullptr)
      return cwm_fail("sample_static: the scratch array has no address on device %d: %s", device, hipGetErrorString(err));
    sample_scratch_ptr[device] = (float*)found;
  }
  *out = sample_scratch_ptr[device];
  return 0;
}

extern "C" int cwm_sample_static_init() {
  float* scratch = nullptr;
  return sample_scratch_on_current_device(&scratch);
}

extern "C" int cwm_sample_static(const float* logits, long row_stride, int n_rows, int vocab,
                                 const float* temperature, const float* top_p, const float* uniform,
                                 int* token_out, float* logprob_out, float* sample_logprob_out,
                                 hipStream_t stream) {
  CWM_REQUIRE(n_rows >= 0 && vocab > 0, "sample_static: bad sizes rows=%d vocab=%d", n_rows, vocab);
  CWM_REQUIRE(row_stride >= vocab, "sample_static: row stride shorter than the vocabulary");
  CWM_REQUIRE((long long)n_rows * vocab <= (long long)CWM_SAMPLE_STATIC_MAX_FLOATS,
              "sample_static: %d rows of %d logits need %lld floats of scratch, the fixed array holds %d", n_rows, vocab,
              (long long)n_rows * vocab, CWM_SAMPLE_STATIC_MAX_FLOATS);
  if (n_rows == 0) return 0;
  float* scratch = nullptr;
  if (int status = sample_scratch_on_current_device(&scratch)) return status;
  launch_sample(logits, row_stride, n_rows, vocab, temperature, top_p, uniform, scratch, token_out, logprob_out, sample_logprob_out, stream);
  return cwm_launch_status("sample_static");
}

// log softmax(logits[rows[i]])[targets[i]] for given tokens: the log-probabilities of a
// prompt's own tokens (cwm/fastgen/forward.py:908-924).  One block per entry.
__global__ void __launch_bounds__(SAMPLE_THREADS)
token_logprob_kernel(const float* __restrict__ logits, long row_stride, int vocab, const int* __restrict__ rows,
                     const int* __restrict__ targets, float* __restrict__ out) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const float* x = logits + (size_t)rows[i] * row_stride;
  float mx = -__builtin_inff();
#pragma unroll 4
  for (int v = threadIdx.x; v < vocab; v += SAMPLE_THREADS) mx = fmaxf(mx, x[v]);
  mx = block_max(mx, scratch);
  float sum = 0.f;
#pragma unroll 4
  for (int v = threadIdx.x; v < vocab; v += SAMPLE_THREADS) sum += expf(x[v] - mx);
  sum = block_sum(sum, scratch);
  if (threadIdx.x == 0) {
    const int t = targets[i];
    out[i] = (t >= 0 && t < vocab) ? x[t] - (mx + logf(sum)) : __uint_as_float(0x7fc00000u);
  }
}

extern "C" int cwm_token_logprob(const float* logits, long row_stride, int n_rows_total, int vocab, const int* rows,
                                 const int* targets, int n, float* out, hipStream_t stream) {
  CWM_REQUIRE(n >= 0 && vocab > 0 && n_rows_total >= 0, "token_logprob: bad sizes");
  CWM_REQUIRE(row_stride >= vocab, "token_logprob: row stride shorter than the vocabulary");
  if (n == 0) return 0;
  hipLaunchKernelGGL(token_logprob_kernel, dim3(n), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride, vocab, rows,
                     targets, out);
  return cwm_launch_status("token_logprob");
}
