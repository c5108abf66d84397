// The sampler: one block per row of float32 logits.
//   greedy (temperature 0 or top_k 1): first index of the maximum, and its
//     log-probability under softmax(logits);
//   otherwise z = logits / temperature, p = softmax(z), the reference's filters
//     (top-k, top-p, min-p), and the first token, in index order, whose cumulative
//     kept probability exceeds u * (kept mass).  u comes from a counter-based
//     generator keyed by (seed, draw index) of the row's request, so a request's
//     tokens do not depend on what else is in the batch.  The log-probability is
//     that of the temperature-scaled distribution before filtering.
// NaN logits count as -1e5.  src/halite/transformers/infer/engine/sampler.py:17-60
#include "hal_common.h"
#include "hal_api.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ float clean_logit(float x) { return x != x ? -1e5f : x; }

// order-preserving map of a float to an unsigned key
__device__ __forceinline__ uint32_t sort_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float uniform_draw(uint64_t seed, uint32_t index) {
  uint64_t x = seed * 0x9E3779B97F4A7C15ull + ((uint64_t)index + 1ull) * 0xD1B54A32D192ED03ull;
  x ^= x >> 30;
  x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27;
  x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  return (float)(x >> 40) * (1.0f / 16777216.0f);
}

struct ArgMax {
  float v;
  int i;
};

__device__ __forceinline__ ArgMax argmax_merge(ArgMax a, ArgMax b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int ld, int V,
              const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ min_p,
              const uint64_t* __restrict__ seeds, const int* __restrict__ draw_index,
              int* __restrict__ out_token, float* __restrict__ out_logprob) {
  __shared__ float red[16];
  __shared__ float red2[16];
  __shared__ ArgMax amax_s[16];
  __shared__ float chunk_sum[SAMPLE_THREADS];
  __shared__ int chosen_thread;
  __shared__ int last_thread;

  const int row = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row];
  const int k = top_k[row];
  const bool greedy = (T == 0.f) || (k == 1);
  const float inv_scale = greedy ? 1.f : T;

  // ---- one pass: maximum (with its first index) and sum of exp(z - max), z = x / T ----
  // Each thread keeps a running maximum and a sum relative to it (the online form of
  // softmax's denominator); four logits per load where the row allows it.
  ArgMax am = {-INFINITY, 0x7fffffff};
  float part = 0.f;
  auto take = [&](float xv, int i) {
    const float z = clean_logit(xv) / inv_scale;
    if (z > am.v) {
      part = part * expf(am.v - z) + 1.f;  // am.v = -inf gives part * 0
      am.v = z;
      am.i = i;
    } else {
      part += expf(z - am.v);
    }
  };
  if (ld % 4 == 0 && ((uintptr_t)logits % 16) == 0) {
    const int n4 = V / 4;
#pragma unroll 4
    for (int v = tid; v < n4; v += SAMPLE_THREADS) {
      const float4 q = *(const float4*)(x + 4 * v);
      take(q.x, 4 * v), take(q.y, 4 * v + 1), take(q.z, 4 * v + 2), take(q.w, 4 * v + 3);
    }
    for (int i = 4 * n4 + tid; i < V; i += SAMPLE_THREADS) take(x[i], i);
  } else {
    for (int i = tid; i < V; i += SAMPLE_THREADS) take(x[i], i);
  }
  // combine the threads: the block's maximum, then the sums rescaled to it
  ArgMax mine_am = am;
#pragma unroll
  for (int off = HAL_WAVE / 2; off > 0; off >>= 1) {
    ArgMax o;
    o.v = __shfl_xor(am.v, off, HAL_WAVE);
    o.i = __shfl_xor(am.i, off, HAL_WAVE);
    am = argmax_merge(am, o);
  }
  if (lane == 0) amax_s[wave] = am;
  __syncthreads();
  am = amax_s[0];
  for (int w = 1; w < SAMPLE_THREADS / HAL_WAVE; ++w) am = argmax_merge(am, amax_s[w]);
  const float m = am.v;
  part = (mine_am.v == -INFINITY) ? 0.f : part * expf(mine_am.v - m);
  const float total = block_sum(part, red);

  if (greedy) {
    if (tid == 0) {
      out_token[row] = am.i;
      out_logprob[row] = -logf(total);  // z_max - m - log(total)
    }
    return;
  }

  // ---- filters: the kept set is { key(z_i) >= key_min } and exp(z_i - m) >= min_p --
  const float tp = top_p[row];
  const float mp = min_p[row];
  uint32_t key_min = 0;
  float ref_mass = total;
  if (k > 0 && k < V) {
    // smallest key with fewer than k elements strictly above it
    uint32_t lo = 0, hi = 0xffffffffu;  // predicate false below the answer, true at hi
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float cnt = 0.f;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const float z = clean_logit(x[i]) / inv_scale;
        if (sort_key(z) > mid) cnt += 1.f;
      }
      cnt = block_sum(cnt, red);
      if (cnt < (float)k) hi = mid; else lo = mid + 1;
    }
    key_min = lo;
    if (mp > 0.f) {
      // with min_p the reference renormalises after top-k, so top-p refers to
      // the mass that top-k kept
      float kept = 0.f;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const float z = clean_logit(x[i]) / inv_scale;
        if (sort_key(z) >= key_min) kept += expf(z - m);
      }
      ref_mass = block_sum(kept, red);
    }
  }
  if (tp < 1.f) {
    // smallest key such that the elements strictly above it hold < top_p of the mass
    const float thr = tp * ref_mass;
    uint32_t lo = 0, hi = 0xffffffffu;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float mass = 0.f;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const float z = clean_logit(x[i]) / inv_scale;
        if (sort_key(z) > mid) mass += expf(z - m);
      }
      mass = block_sum(mass, red2);
      if (mass < thr) hi = mid; else lo = mid + 1;
    }
    if (lo > key_min) key_min = lo;
  }

  // ---- inverse CDF over the kept tokens in index order -----------------------------
  // A thread owns a contiguous run of tokens; a block-wide prefix sum of the runs'
  // kept mass finds the run that holds the target, and its thread walks it.
  const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int begin = tid * chunk;
  const int end = begin + chunk < V ? begin + chunk : V;
  float mine = 0.f;
#pragma unroll 4
  for (int i = begin; i < end; ++i) {
    const float z = clean_logit(x[i]) / inv_scale;
    const float e = expf(z - m);
    if (sort_key(z) >= key_min && e >= mp) mine += e;
  }
  float incl = mine;
#pragma unroll
  for (int off = 1; off < HAL_WAVE; off <<= 1) {
    const float up = __shfl_up(incl, off, HAL_WAVE);
    if (lane >= off) incl += up;
  }
  if (tid == 0) {
    chosen_thread = 0x7fffffff;
    last_thread = -1;
  }
  if (lane == HAL_WAVE - 1) red2[wave] = incl;
  __syncthreads();
  float before = incl - mine, kept_mass = 0.f;
  for (int w = 0; w < SAMPLE_THREADS / HAL_WAVE; ++w) {
    if (w < wave) before += red2[w];
    kept_mass += red2[w];
  }
  const float target = uniform_draw(seeds[row], (uint32_t)draw_index[row]) * kept_mass;
  if (mine > 0.f) {
    atomicMax(&last_thread, tid);
    if (before + mine > target) atomicMin(&chosen_thread, tid);
  }
  __syncthreads();
  int pick = chosen_thread;
  if (pick == 0x7fffffff) pick = last_thread;  // rounding left the target at the very end
  const float chosen_before = before;
  if (tid == pick) {
    float run = chosen_before;
    int tok = -1, last_kept = -1;
    float z_tok = 0.f, z_last = 0.f;
    for (int i = begin; i < end; ++i) {
      const float z = clean_logit(x[i]) / inv_scale;
      const float e = expf(z - m);
      if (sort_key(z) >= key_min && e >= mp) {
        run += e;
        last_kept = i;
        z_last = z;
        if (run > target) {
          tok = i;
          z_tok = z;
          break;
        }
      }
    }
    if (tok < 0) {
      tok = last_kept;
      z_tok = z_last;
    }
    out_token[row] = tok;
    out_logprob[row] = z_tok - m - logf(total);
  }
}

extern "C" int hal_sample(const float* logits, int ld, int n_rows, int V, const float* temperature,
                          const int* top_k, const float* top_p, const float* min_p,
                          const uint64_t* seeds, const int* draw_index, int* out_token,
                          float* out_logprob, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "hal_sample: bad sizes rows=%d V=%d ld=%d", n_rows,
              V, ld);
  if (n_rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, ld, V,
                     temperature, top_k, top_p, min_p, seeds, draw_index, out_token, out_logprob);
  HAL_LAUNCH_CHECK();
  return 0;
}
