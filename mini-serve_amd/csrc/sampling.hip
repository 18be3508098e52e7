// Token selection on the device from float32 logits [rows, vocab]: first-index argmax for greedy
// rows; for sampled rows argmax(logits / T + g) with Gumbel noise g = -log(-log u), u hashed from
// (seed, counter, vocabulary index), and an optional nucleus (top-p) mask applied first. No
// [rows, vocab] temporaries: the noise is computed in registers. One block per row.
#include "common.h"

#define SNT 1024

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x = ((x >> 16) ^ x) * 0x45D9F3Bu;
  x = ((x >> 16) ^ x) * 0x45D9F3Bu;
  return (x >> 16) ^ x;
}

// u in (0, 1): ((h >> 8) + 0.5) * 2^-24 evaluated in float32, kept below 1 (the float32 sum rounds
// the one input 2^24 - 1 up to 2^24, which would make the noise infinite).
__device__ __forceinline__ float hashed_uniform(uint32_t key, uint32_t v) {
  const uint32_t h = mix32(key + v * 0x9E3779B9u);
  const float u = ((float)(h >> 8) + 0.5f) * (1.0f / 16777216.0f);
  return fminf(u, 0.99999994f);
}

struct Best {
  float v;
  int i;
};

__device__ __forceinline__ Best better(Best a, Best b) {  // larger value, then smaller index
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__device__ __forceinline__ Best block_best(Best b, Best* red) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    Best o;
    o.v = __shfl_xor(b.v, off, WAVE);
    o.i = __shfl_xor(b.i, off, WAVE);
    b = better(b, o);
  }
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = b;
  __syncthreads();
  Best t = red[0];
#pragma unroll
  for (int i = 1; i < SNT / WAVE; ++i) t = better(t, red[i]);
  return t;
}

__device__ __forceinline__ float block_sum_s(float v, float* red) { return block_sum<SNT>(v, red); }

__device__ __forceinline__ float block_min(float v, float* red) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v = fminf(v, __shfl_xor(v, off, WAVE));
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < SNT / WAVE; ++i) t = fminf(t, red[i]);
  return t;
}

// temperature / top_p / seed / counter may be null: then every row is greedy.
__global__ __launch_bounds__(SNT) void sample_rows_kernel(const float* __restrict__ logits, int vocab, long long row_stride,
                                                          const float* __restrict__ temperature,
                                                          const float* __restrict__ top_p,
                                                          const unsigned* __restrict__ seed,
                                                          const int* __restrict__ counter, int* __restrict__ tokens) {
  __shared__ Best red_b[SNT / WAVE];
  __shared__ float red_f[SNT / WAVE];
  __shared__ int scan[SNT];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (size_t)row * row_stride;
  const float temp = temperature ? temperature[row] : 0.f;

  if (!(temp > 0.f)) {
    Best b{-INFINITY, 0x7fffffff};
    for (int i = tid; i < vocab; i += SNT) {
      const float v = z[i];
      if (v > b.v) b = Best{v, i};
    }
    b = block_best(b, red_b);
    if (tid == 0) tokens[row] = b.i == 0x7fffffff ? 0 : b.i;
    return;
  }

  const float inv_t = 1.f / temp;
  const uint32_t key = mix32(seed[row] ^ mix32((uint32_t)counter[row]));
  const float nucleus = top_p ? top_p[row] : 1.f;
  float cut = 0.f;     // tokens with probability > cut stay
  int ties_kept = 0;   // and the first ties_kept tokens with probability == cut
  bool masked = nucleus < 1.f;
  float zmax = 0.f, inv_sum = 0.f;

  if (masked) {
    Best b{-INFINITY, 0};
    for (int i = tid; i < vocab; i += SNT) b.v = fmaxf(b.v, z[i] * inv_t);
    zmax = block_best(b, red_b).v;
    float s = 0.f;
    for (int i = tid; i < vocab; i += SNT) s += expf(z[i] * inv_t - zmax);
    inv_sum = 1.f / block_sum_s(s, red_f);
    // Smallest float tau with mass(p > tau) < nucleus, by bisection on the bit pattern.
    uint32_t lo = 0u, hi = __float_as_uint(inv_sum);  // p_max = inv_sum; mass(p > p_max) = 0 < nucleus
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      const float tau = __uint_as_float(mid);
      float m = 0.f;
      for (int i = tid; i < vocab; i += SNT) {
        const float p = expf(z[i] * inv_t - zmax) * inv_sum;
        if (p > tau) m += p;
      }
      m = block_sum_s(m, red_f);
      if (m < nucleus) hi = mid; else lo = mid + 1;
    }
    const float tau = __uint_as_float(lo);
    // The cut is the smallest probability present that is >= tau; its ties stay in index order
    // while the mass before them is below the nucleus.
    float c = INFINITY, above = 0.f;
    for (int i = tid; i < vocab; i += SNT) {
      const float p = expf(z[i] * inv_t - zmax) * inv_sum;
      if (p >= tau) c = fminf(c, p);
    }
    cut = block_min(c, red_f);
    for (int i = tid; i < vocab; i += SNT) {
      const float p = expf(z[i] * inv_t - zmax) * inv_sum;
      if (p > cut) above += p;
    }
    above = block_sum_s(above, red_f);
    // Number of ties kept: ranks k with above + k * cut < nucleus. Estimate, then settle exactly.
    const float est = ceilf((nucleus - above) / cut);
    ties_kept = est >= (float)vocab ? vocab : (est > 0.f ? (int)est : 0);
    while (ties_kept > 0 && !(above + (float)(ties_kept - 1) * cut < nucleus)) --ties_kept;
    while (ties_kept < vocab && above + (float)ties_kept * cut < nucleus) ++ties_kept;
  }

  // Rank of each tie by index needs index order across threads: contiguous chunks per thread.
  const int chunk = (vocab + SNT - 1) / SNT;
  const int begin = tid * chunk, end = min(vocab, begin + chunk);
  int tie_rank = 0;
  if (masked) {
    int mine = 0;
    for (int i = begin; i < end; ++i) mine += (expf(z[i] * inv_t - zmax) * inv_sum == cut);
    scan[tid] = mine;
    __syncthreads();
    for (int off = 1; off < SNT; off <<= 1) {  // inclusive scan
      const int v = tid >= off ? scan[tid - off] : 0;
      __syncthreads();
      scan[tid] += v;
      __syncthreads();
    }
    tie_rank = scan[tid] - mine;
  }

  Best b{-INFINITY, 0x7fffffff};
  for (int i = begin; i < end; ++i) {
    const float zi = z[i] * inv_t;
    if (masked) {
      const float p = expf(zi - zmax) * inv_sum;
      if (p < cut) continue;
      if (p == cut && tie_rank++ >= ties_kept) continue;
    }
    const float u = hashed_uniform(key, (uint32_t)i);
    const float v = zi - logf(-logf(u));
    if (v > b.v) b = Best{v, i};
  }
  b = block_best(b, red_b);
  if (tid == 0) tokens[row] = b.i == 0x7fffffff ? 0 : b.i;
}

extern "C" int ms_sample_rows(const float* logits, int rows, int vocab, long long row_stride, const float* temperature,
                              const float* top_p, const unsigned* seed, const int* counter, int* tokens, hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (vocab <= 0 || row_stride < vocab) return MS_BAD_ARG;
  if (temperature != nullptr && (seed == nullptr || counter == nullptr)) return MS_BAD_ARG;
  sample_rows_kernel<<<rows, SNT, 0, st>>>(logits, vocab, row_stride, temperature, top_p, seed, counter, tokens);
  return launch_status();
}
