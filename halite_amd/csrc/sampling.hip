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
#include <mutex>

#define SAMPLE_THREADS 1024
#define SAMPLE_BINS 2048  // two per thread

__device__ __forceinline__ float clean_logit(float x) { return x != x ? -1e5f : x; }

// order-preserving map of a float to an unsigned key
__device__ __forceinline__ uint32_t sort_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// the float that a key stands for
__device__ __forceinline__ float key_value(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
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

// Sum of `v` over the threads after this one (exclusive), for a block of SAMPLE_THREADS
// threads; `tmp` holds one entry per wave.  Ends with a barrier, so `tmp` can be used
// again at once.
__device__ __forceinline__ unsigned long long block_suffix_u64(unsigned long long v,
                                                               unsigned long long* tmp) {
  const int lane = threadIdx.x % HAL_WAVE, wave = threadIdx.x / HAL_WAVE;
  unsigned long long inc = v;
#pragma unroll
  for (int off = 1; off < HAL_WAVE; off <<= 1) {
    const uint32_t lo = __shfl_down((uint32_t)inc, off, HAL_WAVE);
    const uint32_t hi = __shfl_down((uint32_t)(inc >> 32), off, HAL_WAVE);
    if (lane + off < HAL_WAVE) inc += ((unsigned long long)hi << 32) | lo;
  }
  if (lane == 0) tmp[wave] = inc;
  __syncthreads();
  unsigned long long after = 0ull;
  for (int w = wave + 1; w < SAMPLE_THREADS / HAL_WAVE; ++w) after += tmp[w];
  __syncthreads();
  return inc - v + after;
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
              int* __restrict__ out_token, float* __restrict__ out_logprob,
              uint32_t* __restrict__ key_rows) {
  __shared__ float red[16];
  __shared__ float red2[16];
  __shared__ ArgMax amax_s[16];
  __shared__ int chosen_thread;
  __shared__ int last_thread;
  __shared__ unsigned long long hist[2][SAMPLE_BINS];
  __shared__ unsigned long long scan_tmp[SAMPLE_THREADS / HAL_WAVE];
  __shared__ unsigned long long whole_mass;
  __shared__ unsigned long long found_above[2];
  __shared__ uint32_t found_bin[2];
  __shared__ int found_any[2];

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
  // the keys of the row (order-preserving integers of z) are kept for the later passes
  uint32_t* keys = (key_rows && !greedy) ? key_rows + (size_t)row * V : nullptr;
  auto key_of = [&](float xv) { return sort_key(clean_logit(xv) / inv_scale); };
  auto take = [&](float xv, int i) {
    const float z = clean_logit(xv) / inv_scale;
    if (z > am.v) {
      part = part * expf(am.v - z) + 1.f;  // am.v = -inf gives part * 0
      am.v = z;
      am.i = i;
    } else if (z != -INFINITY) {  // (-inf adds nothing; with am.v still -inf it would add NaN)
      part += expf(z - am.v);
    }
  };
  if (ld % 4 == 0 && ((uintptr_t)logits % 16) == 0) {
    const int n4 = V / 4;
    const bool keys4 = keys && V % 4 == 0;  // rows of keys start on 16 bytes then
#pragma unroll 4
    for (int v = tid; v < n4; v += SAMPLE_THREADS) {
      const float4 q = *(const float4*)(x + 4 * v);
      take(q.x, 4 * v), take(q.y, 4 * v + 1), take(q.z, 4 * v + 2), take(q.w, 4 * v + 3);
      if (keys4)
        *(uint4*)(keys + 4 * v) = make_uint4(key_of(q.x), key_of(q.y), key_of(q.z), key_of(q.w));
      else if (keys)
        keys[4 * v] = key_of(q.x), keys[4 * v + 1] = key_of(q.y), keys[4 * v + 2] = key_of(q.z),
                 keys[4 * v + 3] = key_of(q.w);
    }
    for (int i = 4 * n4 + tid; i < V; i += SAMPLE_THREADS) {
      take(x[i], i);
      if (keys) keys[i] = key_of(x[i]);
    }
  } else {
    for (int i = tid; i < V; i += SAMPLE_THREADS) {
      take(x[i], i);
      if (keys) keys[i] = key_of(x[i]);
    }
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
      out_token[row] = am.i < V ? am.i : 0;  // (a row of nothing but -inf has no maximum)
      out_logprob[row] = -logf(total);  // z_max - m - log(total)
    }
    return;
  }

  // ---- filters: the kept set is { key(z_i) >= key_min } and exp(z_i - m) >= min_p --
  // Both thresholds are the key at which a sum over the tokens in descending order of
  // their keys first reaches a target: the number of tokens reaches k (top-k), the mass
  // reaches top_p of the reference mass (top-p).  That key is found digit by digit
  // (11 + 11 + 10 bits) from histograms over the tokens that share the digits found so
  // far: three passes over the row instead of one per bit.  Masses are summed as
  // integers (2^-40 of the largest token's), so the sums do not depend on their order.
  auto key_at = [&](int i) { return keys ? keys[i] : sort_key(clean_logit(x[i]) / inv_scale); };
  const float tp = top_p[row];
  const float mp = min_p[row];
  const bool want_k = k > 0 && k < V, want_p = tp < 1.f;
  uint32_t key_min = 0;
  if (want_k || want_p) {
    auto fixed = [&](uint32_t key) {
      return (unsigned long long)(expf(key_value(key) - m) * 1099511627776.0f);
    };
    // one search: the digits found so far, the sum over all keys above them, the target
    uint32_t prefix[2] = {0u, 0u};
    unsigned long long above[2] = {0ull, 0ull}, target[2] = {(unsigned long long)(k > 0 ? k : 0), 0ull};
    auto descend = [&](bool on_k, bool on_p) {
      const bool on[2] = {on_k, on_p};
      prefix[0] = on_k ? 0u : prefix[0], prefix[1] = on_p ? 0u : prefix[1];
      above[0] = on_k ? 0ull : above[0], above[1] = on_p ? 0ull : above[1];
#pragma unroll 1
      for (int level = 0; level < 3; ++level) {
        const int shift = level == 0 ? 21 : (level == 1 ? 10 : 0);
        const int up = level == 0 ? 32 : (level == 1 ? 21 : 10);  // bits below `up` are open
        for (int b = tid; b < 2 * SAMPLE_BINS; b += SAMPLE_THREADS) (&hist[0][0])[b] = 0ull;
        __syncthreads();
        for (int i = tid; i < V; i += SAMPLE_THREADS) {
          const uint32_t key = key_at(i);
          const uint32_t high = level == 0 ? 0u : key >> up;
          const uint32_t bin = (key >> shift) & (SAMPLE_BINS - 1) & ((1u << (up - shift)) - 1u);
          if (on[0] && high == prefix[0]) atomicAdd(&hist[0][bin], 1ull);
          if (on[1] && high == prefix[1]) atomicAdd(&hist[1][bin], fixed(key));
        }
        __syncthreads();
        if (level == 0 && on[1]) {
          // the whole mass, as the histogram has it: the reference of top-p unless the
          // caller has set another
          unsigned long long all = hist[1][2 * tid] + hist[1][2 * tid + 1];
          all += block_suffix_u64(all, scan_tmp);
          if (tid == 0) whole_mass = all;
          __syncthreads();
          if (target[1] == ~0ull) {
            const double t = (double)tp * (double)whole_mass;
            target[1] = (unsigned long long)t;
          }
        }
#pragma unroll
        for (int sidx = 0; sidx < 2; ++sidx) {
          if (!on[sidx]) continue;
          // bins in descending order: thread t has bins 2t+1 and 2t
          const unsigned long long h1 = hist[sidx][2 * tid + 1], h0 = hist[sidx][2 * tid];
          const unsigned long long higher = above[sidx] + block_suffix_u64(h1 + h0, scan_tmp);
          if (tid == 0) found_bin[sidx] = 0u, found_above[sidx] = above[sidx] + 0ull, found_any[sidx] = 0;
          __syncthreads();
          if (higher < target[sidx] && higher + h1 >= target[sidx]) {
            found_bin[sidx] = 2 * tid + 1, found_above[sidx] = higher, found_any[sidx] = 1;
          } else if (higher + h1 < target[sidx] && higher + h1 + h0 >= target[sidx]) {
            found_bin[sidx] = 2 * tid, found_above[sidx] = higher + h1, found_any[sidx] = 1;
          }
          __syncthreads();
          // a target of zero, or one beyond the whole sum, is met by no bin: the first
          // keeps the largest key only, the second every key
          if (!found_any[sidx]) {
            if (target[sidx] == 0ull) {
              int top = -1;
              if (h1 != 0ull) top = 2 * tid + 1; else if (h0 != 0ull) top = 2 * tid;
              if (top >= 0) atomicMax(&found_bin[sidx], (uint32_t)top);
            }
            __syncthreads();
          }
          prefix[sidx] = (prefix[sidx] << (up - shift)) | found_bin[sidx];
          above[sidx] = found_above[sidx];
          __syncthreads();
        }
      }
    };
    const bool p_after_k = want_k && want_p && mp > 0.f;  // top-p refers to what top-k kept
    target[1] = ~0ull;                                    // top_p of the whole mass
    if (!p_after_k) {
      descend(want_k, want_p);
      if (want_k) key_min = prefix[0];
      if (want_p && prefix[1] > key_min) key_min = prefix[1];
    } else {
      descend(true, false);
      key_min = prefix[0];
      // with min_p the reference renormalises after top-k, so top-p refers to the
      // mass that top-k kept
      unsigned long long kept = 0ull;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const uint32_t key = key_at(i);
        if (key >= key_min) kept += fixed(key);
      }
      kept += block_suffix_u64(kept, scan_tmp);
      if (tid == 0) whole_mass = kept;
      __syncthreads();
      target[1] = (unsigned long long)((double)tp * (double)whole_mass);
      __syncthreads();
      descend(false, true);
      if (prefix[1] > key_min) key_min = prefix[1];
    }
  }

  // ---- inverse CDF over the kept tokens in index order -----------------------------
  // A wave owns a contiguous run of tokens and reads it 64 tokens at a time; a prefix
  // sum over the waves' kept masses finds the wave that holds the target, and that wave
  // walks its run again with a prefix sum over each 64 tokens.
  const int n_waves = SAMPLE_THREADS / HAL_WAVE;
  const int run_len = ((V + n_waves - 1) / n_waves + HAL_WAVE - 1) / HAL_WAVE * HAL_WAVE;
  const int begin = wave * run_len;
  const int end = begin + run_len < V ? begin + run_len : V;
  auto kept_mass_of = [&](int i, float& z) {
    if (i >= end) return 0.f;
    const uint32_t key = key_at(i);
    if (key < key_min) return 0.f;
    z = key_value(key);
    const float e = expf(z - m);
    return e >= mp ? e : 0.f;
  };
  float mine = 0.f, zz;
  for (int i = begin + lane; i < end; i += HAL_WAVE) mine += kept_mass_of(i, zz);
  const float wave_mass = wave_sum(mine);
  if (tid == 0) {
    chosen_thread = 0x7fffffff;
    last_thread = -1;
  }
  if (lane == 0) red2[wave] = wave_mass;
  __syncthreads();
  float before = 0.f, kept_mass = 0.f;
  for (int w = 0; w < n_waves; ++w) {
    if (w < wave) before += red2[w];
    kept_mass += red2[w];
  }
  const float target = uniform_draw(seeds[row], (uint32_t)draw_index[row]) * kept_mass;
  if (lane == 0 && wave_mass > 0.f) {
    atomicMax(&last_thread, wave);
    if (before + wave_mass > target) atomicMin(&chosen_thread, wave);
  }
  __syncthreads();
  int pick = chosen_thread;
  if (pick == 0x7fffffff) pick = last_thread;  // rounding left the target at the very end
  if (pick < 0) pick = 0;                      // nothing is kept anywhere: token 0 below
  if (wave != pick) return;
  float run = before;
  int tok = -1, last_kept = -1;
  float z_tok = 0.f, z_last = 0.f;
  for (int i0 = begin; i0 < end && tok < 0; i0 += HAL_WAVE) {
    float z = 0.f;
    const float e = kept_mass_of(i0 + lane, z);
    float incl = e;
#pragma unroll
    for (int off = 1; off < HAL_WAVE; off <<= 1) {
      const float up = __shfl_up(incl, off, HAL_WAVE);
      if (lane >= off) incl += up;
    }
    const unsigned long long kept_lanes = __builtin_amdgcn_ballot_w64(e > 0.f);
    const unsigned long long hit = __builtin_amdgcn_ballot_w64(e > 0.f && run + incl > target);
    if (kept_lanes) {
      const int hi = 63 - __builtin_clzll(kept_lanes);
      last_kept = i0 + hi;
      z_last = __shfl(z, hi, HAL_WAVE);
    }
    if (hit) {
      const int lo = __builtin_ctzll(hit);
      tok = i0 + lo;
      z_tok = __shfl(z, lo, HAL_WAVE);
    }
    run += __shfl(incl, HAL_WAVE - 1, HAL_WAVE);
  }
  if (tok < 0) {
    tok = last_kept >= 0 ? last_kept : (am.i < V ? am.i : 0);
    z_tok = last_kept >= 0 ? z_last : m;
  }
  if (lane == 0) {
    out_token[row] = tok;
    out_logprob[row] = z_tok - m - logf(total);
  }
}

// `key_rows`: room for n_rows * V 32-bit words that the kernel may use between its
// passes, or null (every pass then derives the keys from the logits again).
extern "C" int hal_sample(const float* logits, int ld, int n_rows, int V, const float* temperature,
                          const int* top_k, const float* top_p, const float* min_p,
                          const uint64_t* seeds, const int* draw_index, int* out_token,
                          float* out_logprob, uint32_t* key_rows, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "hal_sample: bad sizes rows=%d V=%d ld=%d", n_rows,
              V, ld);
  if (n_rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, ld, V,
                     temperature, top_k, top_p, min_p, seeds, draw_index, out_token, out_logprob,
                     key_rows);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- no row has a filter: the row is spread over ROW_PARTS blocks ---------------------------
// Greedy rows and rows that draw from the whole temperature-scaled distribution need the
// row's maximum, the sum of exp(z - maximum) and, for a draw, one walk to the token at which
// the cumulative probability passes u: no thresholds.  Stage one: a block takes a contiguous
// share of a row and leaves its maximum, the first index of that maximum and the sum of
// exp(z - maximum), z = logit / temperature (the logit itself for a greedy row).  Stage two
// joins a row's shares in order (ties go to the lower index, as everywhere); for a draw it
// finds the share in which the running sum passes u * total and walks that share, a quarter
// per wave, as the one-block kernel walks the row.  Same generator, same rule, same
// log-probability as there; sums are added in another order, so a draw within rounding of a
// token's edge may fall to its neighbour.
#define ROW_PARTS 32
#define PART_THREADS 256

__device__ __forceinline__ int part_share(int V) { return ((V + ROW_PARTS - 1) / ROW_PARTS + 3) / 4 * 4; }
// a row is greedy if it has no temperature array (all rows greedy), a temperature of 0 or top_k 1
__device__ __forceinline__ float row_scale_of(const float* temperature, const int* top_k, int row) {
  if (!temperature) return 0.f;
  const float T = temperature[row];
  return (T == 0.f || (top_k && top_k[row] == 1)) ? 0.f : T;
}

__global__ void __launch_bounds__(PART_THREADS)
row_part_kernel(const float* __restrict__ logits, int ld, int V,
                const float* __restrict__ temperature, const int* __restrict__ top_k,
                float* __restrict__ parts) {
  __shared__ ArgMax amax_s[PART_THREADS / HAL_WAVE];
  __shared__ float red[16];
  const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const int share = part_share(V);
  const int begin = part * share;
  const int end = begin + share < V ? begin + share : V;
  const float* x = logits + (size_t)row * ld;
  const float T = row_scale_of(temperature, top_k, row);
  const float inv_scale = T == 0.f ? 1.f : T;
  ArgMax am = {-INFINITY, 0x7fffffff};
  for (int i = begin + tid; i < end; i += PART_THREADS) {
    const float z = clean_logit(x[i]) / inv_scale;
    if (z > am.v) am.v = z, am.i = i;  // a thread's indices rise: the first maximum stays
  }
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
  for (int w = 1; w < PART_THREADS / HAL_WAVE; ++w) am = argmax_merge(am, amax_s[w]);
  float sum = 0.f;
  for (int i = begin + tid; i < end; i += PART_THREADS) sum += expf(clean_logit(x[i]) / inv_scale - am.v);
  sum = block_sum(sum, red);
  if (tid == 0) {
    float* p = parts + ((size_t)row * ROW_PARTS + part) * 4;
    p[0] = am.v;
    p[1] = __int_as_float(am.i);
    p[2] = begin < end ? sum : 0.f;
  }
}

__global__ void __launch_bounds__(PART_THREADS)
row_join_kernel(const float* __restrict__ logits, int ld, int V, const float* __restrict__ parts,
                const float* __restrict__ temperature, const int* __restrict__ top_k,
                const uint64_t* __restrict__ seeds, const int* __restrict__ draw_index,
                int* __restrict__ out_token, float* __restrict__ out_logprob) {
  __shared__ float quarter_mass[PART_THREADS / HAL_WAVE];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  // every wave joins the shares for itself (32 values)
  ArgMax am = {-INFINITY, 0x7fffffff};
  float sum = 0.f;
  if (lane < ROW_PARTS) {
    const float* p = parts + ((size_t)row * ROW_PARTS + lane) * 4;
    am.v = p[0], am.i = __float_as_int(p[1]), sum = p[2];
  }
  ArgMax best = am;
#pragma unroll
  for (int off = HAL_WAVE / 2; off > 0; off >>= 1) {
    ArgMax o;
    o.v = __shfl_xor(best.v, off, HAL_WAVE);
    o.i = __shfl_xor(best.i, off, HAL_WAVE);
    best = argmax_merge(best, o);
  }
  const float m = best.v;
  const float scaled = (am.v == -INFINITY) ? 0.f : sum * expf(am.v - m);
  const float total = wave_sum(scaled);
  const float T = row_scale_of(temperature, top_k, row);
  if (T == 0.f) {  // greedy
    if (tid == 0) {
      out_token[row] = best.i < V ? best.i : 0;
      out_logprob[row] = -logf(total);
    }
    return;
  }
  // the share in which the running sum (shares in order) passes the target
  const float target = uniform_draw(seeds[row], (uint32_t)draw_index[row]) * total;
  float incl = scaled;
#pragma unroll
  for (int off = 1; off < HAL_WAVE; off <<= 1) {
    const float up = __shfl_up(incl, off, HAL_WAVE);
    if (lane >= off) incl += up;
  }
  const unsigned long long some = __builtin_amdgcn_ballot_w64(scaled > 0.f);
  const unsigned long long hit = __builtin_amdgcn_ballot_w64(scaled > 0.f && incl > target);
  // rounding may leave the target at the very end: the last share that holds anything
  // (a row of nothing but -inf holds nothing anywhere: share 0 then, and token 0 below)
  const int part = hit ? __builtin_ctzll(hit) : (some ? 63 - __builtin_clzll(some) : 0);
  const float before_part = __shfl(incl - scaled, part, HAL_WAVE);

  // the share is walked as the one-block kernel walks a row: a quarter per wave
  const float* x = logits + (size_t)row * ld;
  const int share = part_share(V);
  const int p_begin = part * share, p_end = p_begin + share < V ? p_begin + share : V;
  constexpr int n_waves = PART_THREADS / HAL_WAVE;
  const int run_len = ((p_end - p_begin + n_waves - 1) / n_waves + HAL_WAVE - 1) / HAL_WAVE * HAL_WAVE;
  const int begin = p_begin + wave * run_len;
  const int end = begin + run_len < p_end ? begin + run_len : p_end;
  auto mass_of = [&](int i, float& z) {
    if (i >= end) return 0.f;
    z = clean_logit(x[i]) / T;
    return expf(z - m);
  };
  float mine = 0.f, zz;
  for (int i = begin + lane; i < end; i += HAL_WAVE) mine += mass_of(i, zz);
  const float wave_mass = wave_sum(mine);
  if (lane == 0) quarter_mass[wave] = wave_mass;
  __syncthreads();
  float before = before_part;
  int pick = -1, last = -1;
  for (int w = 0; w < n_waves; ++w) {
    if (quarter_mass[w] > 0.f) last = w;
    if (pick < 0 && quarter_mass[w] > 0.f && before + quarter_mass[w] > target) pick = w;
    if (pick < 0) before += quarter_mass[w];
  }
  if (pick < 0) {  // rounding again: the last quarter that holds anything, from its start
    pick = last < 0 ? 0 : last;
    before = before_part;
    for (int w = 0; w < pick; ++w) before += quarter_mass[w];
  }
  if (wave != pick) return;
  float run = before;
  int tok = -1, last_kept = -1;
  float z_tok = 0.f, z_last = 0.f;
  for (int i0 = begin; i0 < end && tok < 0; i0 += HAL_WAVE) {
    float z = 0.f;
    const float e = mass_of(i0 + lane, z);
    float inc = e;
#pragma unroll
    for (int off = 1; off < HAL_WAVE; off <<= 1) {
      const float up = __shfl_up(inc, off, HAL_WAVE);
      if (lane >= off) inc += up;
    }
    const unsigned long long kept_lanes = __builtin_amdgcn_ballot_w64(e > 0.f);
    const unsigned long long found = __builtin_amdgcn_ballot_w64(e > 0.f && run + inc > target);
    if (kept_lanes) {
      const int hi = 63 - __builtin_clzll(kept_lanes);
      last_kept = i0 + hi;
      z_last = __shfl(z, hi, HAL_WAVE);
    }
    if (found) {
      const int lo = __builtin_ctzll(found);
      tok = i0 + lo;
      z_tok = __shfl(z, lo, HAL_WAVE);
    }
    run += __shfl(inc, HAL_WAVE - 1, HAL_WAVE);
  }
  if (tok < 0) {
    tok = last_kept >= 0 ? last_kept : (best.i < V ? best.i : 0);
    z_tok = last_kept >= 0 ? z_last : m;
  }
  if (lane == 0) {
    out_token[row] = tok;
    out_logprob[row] = z_tok - m - logf(total);
  }
}

// ---- rows with filters, spread over many blocks -----------------------------------------
// The one-block kernel above spends most of its time in the first histogram: a row's keys
// crowd into a few dozen of the 2,048 bins, and a block's atomics on one bin wait for each
// other.  Here a row's keys are split over ROW_PARTS blocks for every pass; a block builds
// its histogram in LDS and adds the bins it has filled to the row's histogram in memory
// (integers: the order does not matter), and a one-block kernel per row walks that histogram
// exactly as the kernel above walks its own.  Thresholds are therefore the same keys as
// there; the drawn token may differ where the draw is within rounding of a token's edge,
// since the kept masses are added in another order.  A row with top-k, top-p and min-p all
// at once, where top-p refers to what top-k kept, is searched twice: top-k first, then (the
// `late` passes) the mass that top-k kept and top-p within it.
struct FiltRow {
  float m, total;  // maximum of z and sum of exp(z - m) over the row
  int best;        // first index of the maximum
  int flags;       // FILT_*
  uint32_t prefix[2];
  uint32_t key_min;
  uint32_t unused;
  unsigned long long above[2], target[2];
  unsigned long long kept_by_k;  // late rows: the mass of the keys that top-k kept
  unsigned long long unused2;
};
static_assert(sizeof(FiltRow) == 80, "FiltRow is 20 words");
// greedy; top-k is searched; top-p is searched beside it; top-p is searched after it (late)
enum { FILT_GREEDY = 1, FILT_K = 2, FILT_P = 4, FILT_P_LATE = 8 };

__device__ __forceinline__ int level_shift(int level) { return level == 0 ? 21 : (level == 1 ? 10 : 0); }
__device__ __forceinline__ int level_up(int level) { return level == 0 ? 32 : (level == 1 ? 21 : 10); }

__global__ void __launch_bounds__(HAL_WAVE)
filt_join_kernel(const float* __restrict__ parts, const float* __restrict__ temperature,
                 const int* __restrict__ top_k, const float* __restrict__ top_p,
                 const float* __restrict__ min_p, int V, FiltRow* __restrict__ rows,
                 unsigned long long* __restrict__ hist) {
  const int row = blockIdx.x, lane = threadIdx.x;
  // the row's histogram starts at zero (the searches leave it so, but the room may be new)
  for (int b = lane; b < 2 * SAMPLE_BINS; b += HAL_WAVE) hist[(size_t)row * 2 * SAMPLE_BINS + b] = 0ull;
  ArgMax am = {-INFINITY, 0x7fffffff};
  float sum = 0.f;
  if (lane < ROW_PARTS) {
    const float* p = parts + ((size_t)row * ROW_PARTS + lane) * 4;
    am.v = p[0], am.i = __float_as_int(p[1]), sum = p[2];
  }
  ArgMax best = am;
#pragma unroll
  for (int off = HAL_WAVE / 2; off > 0; off >>= 1) {
    ArgMax o;
    o.v = __shfl_xor(best.v, off, HAL_WAVE);
    o.i = __shfl_xor(best.i, off, HAL_WAVE);
    best = argmax_merge(best, o);
  }
  const float scaled = (am.v == -INFINITY) ? 0.f : sum * expf(am.v - best.v);
  const float total = wave_sum(scaled);
  if (lane != 0) return;
  const bool greedy = row_scale_of(temperature, top_k, row) == 0.f;
  const int k = top_k[row];
  FiltRow r;
  r.m = best.v, r.total = total, r.best = best.i;
  const bool want_k = k > 0 && k < V, want_p = top_p[row] < 1.f;
  // with min_p the reference renormalises after top-k, so top-p refers to what top-k kept
  const bool late = want_k && want_p && min_p[row] > 0.f;
  r.flags = greedy ? FILT_GREEDY : ((want_k ? FILT_K : 0) | (want_p ? (late ? FILT_P_LATE : FILT_P) : 0));
  r.prefix[0] = r.prefix[1] = 0u, r.key_min = 0u, r.unused = 0u, r.kept_by_k = 0ull, r.unused2 = 0ull;
  r.above[0] = r.above[1] = 0ull;
  r.target[0] = (unsigned long long)(k > 0 ? k : 0), r.target[1] = ~0ull;  // top_p of the whole mass, set at level 0
  rows[row] = r;
}

// One level of the search: the histogram of a share of the row, added to the row's.
__global__ void __launch_bounds__(PART_THREADS)
filt_hist_kernel(const float* __restrict__ logits, int ld, int V,
                 const float* __restrict__ temperature, const FiltRow* __restrict__ rows, int level,
                 int late, unsigned long long* __restrict__ hist) {  // [rows][2][SAMPLE_BINS]
  __shared__ uint32_t count_s[SAMPLE_BINS];
  __shared__ unsigned long long mass_s[SAMPLE_BINS];
  const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
  const FiltRow r = rows[row];
  const bool on_k = !late && (r.flags & FILT_K) != 0;
  const bool on_p = (r.flags & (late ? FILT_P_LATE : FILT_P)) != 0;
  if (!on_k && !on_p) return;
  for (int b = tid; b < SAMPLE_BINS; b += PART_THREADS) count_s[b] = 0u, mass_s[b] = 0ull;
  __syncthreads();
  const int share = part_share(V);
  const int begin = part * share, end = begin + share < V ? begin + share : V;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row];
  const int shift = level_shift(level), up = level_up(level);
  for (int i = begin + tid; i < end; i += PART_THREADS) {
    const uint32_t key = sort_key(clean_logit(x[i]) / T);
    const uint32_t high = level == 0 ? 0u : key >> up;
    const uint32_t bin = (key >> shift) & (SAMPLE_BINS - 1) & ((1u << (up - shift)) - 1u);
    if (on_k && high == r.prefix[0]) atomicAdd(&count_s[bin], 1u);
    if (on_p && high == r.prefix[1])
      atomicAdd(&mass_s[bin], (unsigned long long)(expf(key_value(key) - r.m) * 1099511627776.0f));
  }
  __syncthreads();
  unsigned long long* h = hist + (size_t)row * 2 * SAMPLE_BINS;
  for (int b = tid; b < SAMPLE_BINS; b += PART_THREADS) {
    if (count_s[b]) atomicAdd(&h[b], (unsigned long long)count_s[b]);
    if (mass_s[b]) atomicAdd(&h[SAMPLE_BINS + b], mass_s[b]);
  }
}

// The walk over the row's histogram of one level (as in sample_kernel); leaves the
// histogram cleared for the next level, and after the last level the smallest kept key.
__global__ void __launch_bounds__(SAMPLE_THREADS)
filt_find_kernel(FiltRow* __restrict__ rows, unsigned long long* __restrict__ hist,
                 const float* __restrict__ top_p, int level, int late) {
  __shared__ unsigned long long scan_tmp[SAMPLE_THREADS / HAL_WAVE];
  __shared__ unsigned long long whole_mass;
  __shared__ unsigned long long found_above[2];
  __shared__ uint32_t found_bin[2];
  __shared__ int found_any[2];
  const int row = blockIdx.x, tid = threadIdx.x;
  FiltRow r = rows[row];
  const bool on[2] = {!late && (r.flags & FILT_K) != 0, (r.flags & (late ? FILT_P_LATE : FILT_P)) != 0};
  if (!on[0] && !on[1]) return;
  unsigned long long* h = hist + (size_t)row * 2 * SAMPLE_BINS;
  const int shift = level_shift(level), up = level_up(level);
  if (level == 0 && late) {
    // top-p of what top-k kept
    r.target[1] = (unsigned long long)((double)top_p[row] * (double)r.kept_by_k);
  } else if (level == 0 && on[1]) {
    // the whole mass, as the histogram has it: the reference of top-p
    unsigned long long all = h[SAMPLE_BINS + 2 * tid] + h[SAMPLE_BINS + 2 * tid + 1];
    all += block_suffix_u64(all, scan_tmp);
    if (tid == 0) whole_mass = all;
    __syncthreads();
    r.target[1] = (unsigned long long)((double)top_p[row] * (double)whole_mass);
  }
#pragma unroll
  for (int sidx = 0; sidx < 2; ++sidx) {
    if (!on[sidx]) continue;
    // bins in descending order: thread t has bins 2t+1 and 2t
    const unsigned long long h1 = h[sidx * SAMPLE_BINS + 2 * tid + 1], h0 = h[sidx * SAMPLE_BINS + 2 * tid];
    const unsigned long long higher = r.above[sidx] + block_suffix_u64(h1 + h0, scan_tmp);
    if (tid == 0) found_bin[sidx] = 0u, found_above[sidx] = r.above[sidx], found_any[sidx] = 0;
    __syncthreads();
    if (higher < r.target[sidx] && higher + h1 >= r.target[sidx]) {
      found_bin[sidx] = 2 * tid + 1, found_above[sidx] = higher, found_any[sidx] = 1;
    } else if (higher + h1 < r.target[sidx] && higher + h1 + h0 >= r.target[sidx]) {
      found_bin[sidx] = 2 * tid, found_above[sidx] = higher + h1, found_any[sidx] = 1;
    }
    __syncthreads();
    // a target of zero, or one beyond the whole sum, is met by no bin: the first keeps the
    // largest key only, the second every key
    if (!found_any[sidx]) {
      if (r.target[sidx] == 0ull) {
        int top = -1;
        if (h1 != 0ull) top = 2 * tid + 1; else if (h0 != 0ull) top = 2 * tid;
        if (top >= 0) atomicMax(&found_bin[sidx], (uint32_t)top);
      }
      __syncthreads();
    }
    r.prefix[sidx] = (r.prefix[sidx] << (up - shift)) | found_bin[sidx];
    r.above[sidx] = found_above[sidx];
    __syncthreads();
  }
  // cleared for the next level (every thread has read its bins)
  h[2 * tid] = h[2 * tid + 1] = 0ull;
  h[SAMPLE_BINS + 2 * tid] = h[SAMPLE_BINS + 2 * tid + 1] = 0ull;
  if (tid == 0) {
    if (level == 2) {
      if (!late) r.key_min = on[0] ? r.prefix[0] : 0u;
      if (on[1] && r.prefix[1] > r.key_min) r.key_min = r.prefix[1];
    }
    rows[row] = r;
  }
}

// Late rows: the mass of the keys that top-k kept, as the histograms count it (integers).
__global__ void __launch_bounds__(PART_THREADS)
filt_kept_by_k_kernel(const float* __restrict__ logits, int ld, int V,
                      const float* __restrict__ temperature, FiltRow* __restrict__ rows) {
  __shared__ unsigned long long tmp[PART_THREADS / HAL_WAVE];
  const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const FiltRow r = rows[row];
  if (!(r.flags & FILT_P_LATE)) return;
  const int share = part_share(V);
  const int begin = part * share, end = begin + share < V ? begin + share : V;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row];
  unsigned long long mine = 0ull;
  for (int i = begin + tid; i < end; i += PART_THREADS) {
    const uint32_t key = sort_key(clean_logit(x[i]) / T);
    if (key >= r.key_min) mine += (unsigned long long)(expf(key_value(key) - r.m) * 1099511627776.0f);
  }
#pragma unroll
  for (int off = HAL_WAVE / 2; off > 0; off >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)mine, off, HAL_WAVE);
    const uint32_t hi = __shfl_xor((uint32_t)(mine >> 32), off, HAL_WAVE);
    mine += ((unsigned long long)hi << 32) | lo;
  }
  if (lane == 0) tmp[wave] = mine;
  __syncthreads();
  if (tid == 0) {
    unsigned long long all = 0ull;
    for (int w = 0; w < PART_THREADS / HAL_WAVE; ++w) all += tmp[w];
    if (all) atomicAdd(&rows[row].kept_by_k, all);
  }
}

__device__ __forceinline__ float kept_mass_at(const float* x, int i, float T, const FiltRow& r, float mp,
                                              float& z) {
  const uint32_t key = sort_key(clean_logit(x[i]) / T);
  if (key < r.key_min) return 0.f;
  z = key_value(key);
  const float e = expf(z - r.m);
  return e >= mp ? e : 0.f;
}

// The kept mass of every share of a row.
__global__ void __launch_bounds__(PART_THREADS)
filt_mass_kernel(const float* __restrict__ logits, int ld, int V,
                 const float* __restrict__ temperature, const float* __restrict__ min_p,
                 const FiltRow* __restrict__ rows, float* __restrict__ kept) {  // [rows][ROW_PARTS]
  __shared__ float red[16];
  const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
  const FiltRow r = rows[row];
  if (r.flags & FILT_GREEDY) return;
  const int share = part_share(V);
  const int begin = part * share, end = begin + share < V ? begin + share : V;
  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row], mp = min_p[row];
  float mine = 0.f, z;
  for (int i = begin + tid; i < end; i += PART_THREADS) mine += kept_mass_at(x, i, T, r, mp, z);
  mine = block_sum(mine, red);
  if (tid == 0) kept[(size_t)row * ROW_PARTS + part] = mine;
}

// The draw: the share in which the running kept mass passes u * (kept mass), then the walk
// through that share, a quarter per wave.
__global__ void __launch_bounds__(PART_THREADS)
filt_pick_kernel(const float* __restrict__ logits, int ld, int V,
                 const float* __restrict__ temperature, const float* __restrict__ min_p,
                 const FiltRow* __restrict__ rows, const float* __restrict__ kept,
                 const uint64_t* __restrict__ seeds, const int* __restrict__ draw_index,
                 int* __restrict__ out_token, float* __restrict__ out_logprob) {
  __shared__ float quarter_mass[PART_THREADS / HAL_WAVE];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const FiltRow r = rows[row];
  if (r.flags & FILT_GREEDY) {
    if (tid == 0) {
      out_token[row] = r.best < V ? r.best : 0;
      out_logprob[row] = -logf(r.total);
    }
    return;
  }
  const float mass = lane < ROW_PARTS ? kept[(size_t)row * ROW_PARTS + lane] : 0.f;
  float incl = mass;
#pragma unroll
  for (int off = 1; off < HAL_WAVE; off <<= 1) {
    const float up = __shfl_up(incl, off, HAL_WAVE);
    if (lane >= off) incl += up;
  }
  const float kept_mass = __shfl(incl, HAL_WAVE - 1, HAL_WAVE);
  const float target = uniform_draw(seeds[row], (uint32_t)draw_index[row]) * kept_mass;
  const unsigned long long some = __builtin_amdgcn_ballot_w64(mass > 0.f);
  const unsigned long long hit = __builtin_amdgcn_ballot_w64(mass > 0.f && incl > target);
  // (the largest key is always kept, so some share holds something)
  const int part = hit ? __builtin_ctzll(hit) : (some ? 63 - __builtin_clzll(some) : 0);
  const float before_part = __shfl(incl - mass, part, HAL_WAVE);

  const float* x = logits + (size_t)row * ld;
  const float T = temperature[row], mp = min_p[row];
  const int share = part_share(V);
  const int p_begin = part * share, p_end = p_begin + share < V ? p_begin + share : V;
  constexpr int n_waves = PART_THREADS / HAL_WAVE;
  const int run_len = ((p_end - p_begin + n_waves - 1) / n_waves + HAL_WAVE - 1) / HAL_WAVE * HAL_WAVE;
  const int begin = p_begin + wave * run_len;
  const int end = begin + run_len < p_end ? begin + run_len : p_end;
  float mine = 0.f, zz = 0.f;
  for (int i = begin + lane; i < end; i += HAL_WAVE) mine += kept_mass_at(x, i, T, r, mp, zz);
  const float wave_mass = wave_sum(mine);
  if (lane == 0) quarter_mass[wave] = wave_mass;
  __syncthreads();
  float before = before_part;
  int pick = -1, last = -1;
  for (int w = 0; w < n_waves; ++w) {
    if (quarter_mass[w] > 0.f) last = w;
    if (pick < 0 && quarter_mass[w] > 0.f && before + quarter_mass[w] > target) pick = w;
    if (pick < 0) before += quarter_mass[w];
  }
  if (pick < 0) {  // rounding left the target at the very end: the last quarter that holds anything
    pick = last < 0 ? 0 : last;
    before = before_part;
    for (int w = 0; w < pick; ++w) before += quarter_mass[w];
  }
  if (wave != pick) return;
  float run = before;
  int tok = -1, last_kept = -1;
  float z_tok = 0.f, z_last = 0.f;
  for (int i0 = begin; i0 < end && tok < 0; i0 += HAL_WAVE) {
    float z = 0.f;
    const float e = i0 + lane < end ? kept_mass_at(x, i0 + lane, T, r, mp, z) : 0.f;
    float inc = e;
#pragma unroll
    for (int off = 1; off < HAL_WAVE; off <<= 1) {
      const float up = __shfl_up(inc, off, HAL_WAVE);
      if (lane >= off) inc += up;
    }
    const unsigned long long kept_lanes = __builtin_amdgcn_ballot_w64(e > 0.f);
    const unsigned long long found = __builtin_amdgcn_ballot_w64(e > 0.f && run + inc > target);
    if (kept_lanes) {
      const int hi = 63 - __builtin_clzll(kept_lanes);
      last_kept = i0 + hi;
      z_last = __shfl(z, hi, HAL_WAVE);
    }
    if (found) {
      const int lo = __builtin_ctzll(found);
      tok = i0 + lo;
      z_tok = __shfl(z, lo, HAL_WAVE);
    }
    run += __shfl(inc, HAL_WAVE - 1, HAL_WAVE);
  }
  if (tok < 0) {
    tok = last_kept >= 0 ? last_kept : (r.best < V ? r.best : 0);
    z_tok = last_kept >= 0 ? z_last : r.m;
  }
  if (lane == 0) {
    out_token[row] = tok;
    out_logprob[row] = z_tok - r.m - logf(r.total);
  }
}

static int launch_row_parts(const float* logits, int ld, int n_rows, int V, const float* temperature,
                            const int* top_k, const uint64_t* seeds, const int* draw_index,
                            float* parts, int* out_token, float* out_logprob, hipStream_t stream) {
  hipLaunchKernelGGL(row_part_kernel, dim3(ROW_PARTS, n_rows), dim3(PART_THREADS), 0, stream, logits,
                     ld, V, temperature, top_k, parts);
  HAL_LAUNCH_CHECK();
  hipLaunchKernelGGL(row_join_kernel, dim3(n_rows), dim3(PART_THREADS), 0, stream, logits, ld, V,
                     parts, temperature, top_k, seeds, draw_index, out_token, out_logprob);
  HAL_LAUNCH_CHECK();
  return 0;
}

// Greedy decoding of every row: first index of the maximum and its log-probability under
// softmax(logits).  `parts` has room for n_rows * 32 * 4 floats.
extern "C" int hal_sample_greedy(const float* logits, int ld, int n_rows, int V, float* parts,
                                 int* out_token, float* out_logprob, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "hal_sample_greedy: bad sizes rows=%d V=%d ld=%d",
              n_rows, V, ld);
  HAL_REQUIRE(n_rows <= 65535, "hal_sample_greedy: %d rows exceed the grid limit", n_rows);
  if (n_rows == 0) return 0;
  HAL_REQUIRE(parts != nullptr, "hal_sample_greedy: no room for the partial results");
  return launch_row_parts(logits, ld, n_rows, V, nullptr, nullptr, nullptr, nullptr, parts, out_token,
                          out_logprob, stream);
}

// ---- greedy decoding without any allocation ---------------------------------------------
// The partial results of hal_sample_greedy in memory that the library itself holds: one
// array per GPU, there from the moment the library is loaded until the process ends.
#define STATIC_GREEDY_ROWS 1024
static __device__ __align__(256) float scratch[STATIC_GREEDY_ROWS * ROW_PARTS * 4];  // 512 KiB

#define STATIC_MAX_DEVICES 64
static float* g_scratch_of_device[STATIC_MAX_DEVICES];  // the array's address on each GPU
static std::mutex g_scratch_lock;

// The address of this GPU's copy of `scratch`.  The array's name means nothing to host
// code; the address is asked for once per device, with that device current.
static int scratch_of_current_device(float** out) {
  int dev = -1;
  HAL_CHECK_HIP(hipGetDevice(&dev));
  HAL_REQUIRE(dev >= 0 && dev < STATIC_MAX_DEVICES, "hal_sample_greedy_static: device %d of at most %d",
              dev, STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (g_scratch_of_device[dev] == nullptr) {
    float* ptr = nullptr;
    HAL_CHECK_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    HAL_REQUIRE(ptr != nullptr, "hal_sample_greedy_static: the scratch array has no address on device %d", dev);
    g_scratch_of_device[dev] = ptr;
  }
  *out = g_scratch_of_device[dev];
  return 0;
}

extern "C" int hal_sample_greedy_static_max_rows() { return STATIC_GREEDY_ROWS; }

// hal_sample_greedy for callers that cannot allocate: the partial results go to the
// library's own array on the current GPU instead of to `parts`.  Calls no hipMalloc, no
// hipFree and no routine that allocates; launches the same two kernels.  Nothing in the
// array has to start at zero: the first kernel writes every word that the second reads (32
// shares of every row), so what an earlier call left does no harm.  All calls on a GPU
// share the array: two calls whose kernels may overlap (different streams, different host
// threads) race; calls on one stream follow each other and are safe.
extern "C" int hal_sample_greedy_static(const float* logits, int ld, int n_rows, int V,
                                        int* out_token, float* out_logprob, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "hal_sample_greedy_static: bad sizes rows=%d V=%d ld=%d",
              n_rows, V, ld);
  HAL_REQUIRE(n_rows <= STATIC_GREEDY_ROWS,
              "hal_sample_greedy_static: %d rows, the scratch array holds the partial results of at most %d",
              n_rows, STATIC_GREEDY_ROWS);
  if (n_rows == 0) return 0;
  HAL_REQUIRE(logits && out_token && out_logprob, "hal_sample_greedy_static: arguments missing");
  float* parts = nullptr;
  if (int rc = scratch_of_current_device(&parts)) return rc;
  return launch_row_parts(logits, ld, n_rows, V, nullptr, nullptr, nullptr, nullptr, parts, out_token,
                          out_logprob, stream);
}

// Rows without filters (no top-k beyond 1, no top-p, no min-p): greedy rows (temperature 0
// or top_k 1) and draws from the whole temperature-scaled distribution, as hal_sample gives
// them.  `parts` has room for n_rows * 32 * 4 floats.
extern "C" int hal_sample_unfiltered(const float* logits, int ld, int n_rows, int V,
                                     const float* temperature, const int* top_k,
                                     const uint64_t* seeds, const int* draw_index, float* parts,
                                     int* out_token, float* out_logprob, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "hal_sample_unfiltered: bad sizes rows=%d V=%d ld=%d",
              n_rows, V, ld);
  HAL_REQUIRE(n_rows <= 65535, "hal_sample_unfiltered: %d rows exceed the grid limit", n_rows);
  if (n_rows == 0) return 0;
  HAL_REQUIRE(parts && temperature && top_k && seeds && draw_index,
              "hal_sample_unfiltered: arguments missing");
  return launch_row_parts(logits, ld, n_rows, V, temperature, top_k, seeds, draw_index, parts,
                          out_token, out_logprob, stream);
}

// Rows with filters (and greedy or unfiltered ones among them), every row spread over 32
// blocks in every pass.  `any_late`: some row has top-k, top-p and min-p all at once (its
// second search costs seven launches more; a wrong 0 leaves such a row without top-p).
// Room: `parts` n_rows * 32 * 4 floats, `kept` n_rows * 32 floats, `state` n_rows * 20
// words, `hist` n_rows * 2 * 2048 64-bit words.
extern "C" int hal_sample_spread(const float* logits, int ld, int n_rows, int V,
                                 const float* temperature, const int* top_k, const float* top_p,
                                 const float* min_p, const uint64_t* seeds, const int* draw_index,
                                 float* parts, float* kept, void* state, void* hist, int any_late,
                                 int* out_token, float* out_logprob, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "hal_sample_spread: bad sizes rows=%d V=%d ld=%d",
              n_rows, V, ld);
  HAL_REQUIRE(n_rows <= 65535, "hal_sample_spread: %d rows exceed the grid limit", n_rows);
  if (n_rows == 0) return 0;
  HAL_REQUIRE(temperature && top_k && top_p && min_p && seeds && draw_index && parts && kept &&
                  state && hist && ((uintptr_t)state % 8) == 0 && ((uintptr_t)hist % 8) == 0,
              "hal_sample_spread: arguments missing");
  FiltRow* rows = (FiltRow*)state;
  unsigned long long* h = (unsigned long long*)hist;
  hipLaunchKernelGGL(row_part_kernel, dim3(ROW_PARTS, n_rows), dim3(PART_THREADS), 0, stream, logits,
                     ld, V, temperature, top_k, parts);
  hipLaunchKernelGGL(filt_join_kernel, dim3(n_rows), dim3(HAL_WAVE), 0, stream, parts, temperature,
                     top_k, top_p, min_p, V, rows, h);
  // the searches; then, if some row has top-k, top-p and min-p all at once, its second search
  for (int late = 0; late <= (any_late ? 1 : 0); ++late) {
    if (late)
      hipLaunchKernelGGL(filt_kept_by_k_kernel, dim3(ROW_PARTS, n_rows), dim3(PART_THREADS), 0,
                         stream, logits, ld, V, temperature, rows);
    for (int level = 0; level < 3; ++level) {
      hipLaunchKernelGGL(filt_hist_kernel, dim3(ROW_PARTS, n_rows), dim3(PART_THREADS), 0, stream,
                         logits, ld, V, temperature, rows, level, late, h);
      hipLaunchKernelGGL(filt_find_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, rows, h,
                         top_p, level, late);
    }
  }
  hipLaunchKernelGGL(filt_mass_kernel, dim3(ROW_PARTS, n_rows), dim3(PART_THREADS), 0, stream, logits,
                     ld, V, temperature, min_p, rows, kept);
  hipLaunchKernelGGL(filt_pick_kernel, dim3(n_rows), dim3(PART_THREADS), 0, stream, logits, ld, V,
                     temperature, min_p, rows, kept, seeds, draw_index, out_token, out_logprob);
  HAL_LAUNCH_CHECK();
  return 0;
}
