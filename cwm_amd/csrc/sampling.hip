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
// with f(t*) <= top_p * sum(e); t* is found by bisection on the bit pattern.
// Entries exactly equal to the threshold are all kept.
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

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, long row_stride, int vocab, const float* __restrict__ temperature,
              const float* __restrict__ top_p, const float* __restrict__ uniform, float* __restrict__ workspace,
              int* __restrict__ token_out, float* __restrict__ logprob_out, float* __restrict__ sample_logprob_out) {
  __shared__ float scratch[16];
  __shared__ float mv[SAMPLE_THREADS / CWM_WAVE];
  __shared__ int mi[SAMPLE_THREADS / CWM_WAVE];
  __shared__ float seg_sum[SAMPLE_THREADS];
  __shared__ int chosen_thread;
  __shared__ float chosen_prefix;
  __shared__ float kept_total;
  __shared__ int result_token;
  __shared__ float result_e;

  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float* x = logits + (size_t)row * row_stride;
  float* e = workspace + (size_t)row * vocab;

  // 1. maximum and its first index
  MaxIdx best = {-__builtin_inff(), 0x7fffffff};
#pragma unroll 4
  for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
    const float v = x[i];
    if (v > best.v) {  // strided scan visits indices in increasing order per thread
      best.v = v;
      best.i = i;
    }
  }
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
#pragma unroll 4
  for (int i = tid; i < vocab; i += SAMPLE_THREADS) s1 += expf(x[i] - xmax);
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

  // 3. unnormalised probabilities at temperature T
  const float inv_t = 1.0f / temp;
  float z = 0.f;
#pragma unroll 4
  for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
    const float ev = expf((x[i] - xmax) * inv_t);
    e[i] = ev;
    z += ev;
  }
  z = block_sum(z, scratch);

  // 4. nucleus threshold
  float thresh = 0.f;
  const float tp = top_p[row];
  if (tp < 1.0f) {
    const float target = tp * z;
    uint32_t lo = 0u, hi = __float_as_uint(1.0f);
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      const float t = __uint_as_float(mid);
      float above = 0.f;
#pragma unroll 4
      for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
        const float ev = e[i];
        above += ev > t ? ev : 0.f;
      }
      above = block_sum(above, scratch);
      if (above <= target)
        hi = mid;
      else
        lo = mid + 1;
    }
    thresh = __uint_as_float(hi);
  }

  // 5. inverse CDF over the kept entries in vocabulary order
  const int seg = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int begin = min(vocab, tid * seg);
  const int end = min(vocab, begin + seg);
  float local = 0.f;
  for (int i = begin; i < end; ++i) {
    const float ev = e[i];
    local += ev >= thresh ? ev : 0.f;
  }
  seg_sum[tid] = local;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int i = 0; i < SAMPLE_THREADS; ++i) total += seg_sum[i];
    const float target = uniform[row] * total;
    float run = 0.f;
    int pick = -1;
    float pick_prefix = 0.f;
    int last_nonempty = 0;
    float last_prefix = 0.f;
    for (int i = 0; i < SAMPLE_THREADS; ++i) {
      const float sgm = seg_sum[i];
      if (sgm > 0.f) {
        last_nonempty = i;
        last_prefix = run;
        if (pick < 0 && run + sgm > target) {
          pick = i;
          pick_prefix = run;
        }
      }
      run += sgm;
    }
    if (pick < 0) {  // rounding left the target at or beyond the total
      pick = last_nonempty;
      pick_prefix = last_prefix;
    }
    chosen_thread = pick;
    chosen_prefix = pick_prefix;
    kept_total = total;
  }
  __syncthreads();
  if (tid == chosen_thread) {
    const float target = uniform[row] * kept_total;
    float run = chosen_prefix;
    int tok = -1;
    float tok_e = 0.f;
    for (int i = begin; i < end; ++i) {
      const float ev = e[i];
      if (ev >= thresh && ev > 0.f) {
        tok = i;  // remembers the last kept entry in case rounding overshoots
        tok_e = ev;
        run += ev;
        if (run > target) break;
      }
    }
    result_token = tok;
    result_e = tok_e;
  }
  __syncthreads();
  if (tid == 0) {
    const int tok = result_token >= 0 ? result_token : best.i;
    token_out[row] = tok;
    logprob_out[row] = x[tok] - lse;
    sample_logprob_out[row] = logf(result_e / kept_total);
  }
}

extern "C" int cwm_sample(const float* logits, long row_stride, int n_rows, int vocab, const float* temperature,
                          const float* top_p, const float* uniform, float* workspace, int* token_out,
                          float* logprob_out, float* sample_logprob_out, hipStream_t stream) {
  CWM_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", n_rows, vocab);
  CWM_REQUIRE(row_stride >= vocab, "sample: row stride shorter than the vocabulary");
  CWM_REQUIRE(workspace != nullptr, "sample: workspace missing");
  if (n_rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride, vocab,
                     temperature, top_p, uniform, workspace, token_out, logprob_out, sample_logprob_out);
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
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return cwm_fail("sample_static: hipGetDevice failed: %s", hipGetErrorString(err));
  CWM_REQUIRE(device >= 0 && device < CWM_MAX_DEVICES, "sample_static: device %d is outside 0..%d", device, CWM_MAX_DEVICES - 1);
  float* scratch = nullptr;
  {
    std::lock_guard<std::mutex> guard(sample_scratch_mutex);
    if (sample_scratch_ptr[device] == nullptr) {
      void* found = nullptr;
      err = hipGetSymbolAddress(&found, HIP_SYMBOL(sample_scratch));
      if (err != hipSuccess || found == nullptr)
        return cwm_fail("sample_static: the scratch array has no address on device %d: %s", device, hipGetErrorString(err));
      sample_scratch_ptr[device] = (float*)found;
    }
    scratch = sample_scratch_ptr[device];
  }
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride, vocab,
                     temperature, top_p, uniform, scratch, token_out, logprob_out, sample_logprob_out);
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
