// Token selection on the device from float32 logits [rows, vocab]: first-index argmax for greedy
// rows; for sampled rows argmax(logits / T + g) with Gumbel noise g = -log(-log u), u hashed from
// (seed, counter, vocabulary index), and an optional nucleus (top-p) mask applied first. No
// [rows, vocab] temporaries: the noise is computed in registers. Rows without a nucleus (greedy, or
// plain temperature) are searched by SPARTS blocks each, whose best candidates a second kernel
// compares; that second kernel also does the rows with a nucleus, one block per row, whole.
#include "common.h"
#include "sampling.h"
#include <mutex>

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

#define SPARTS 64  // blocks per row in the first kernel
#define SPT 256    // threads of such a block

// First kernel, grid (rows, SPARTS): the best candidate of a contiguous part of the vocabulary for
// rows without a nucleus: the largest logit (greedy), or the largest logit / T + noise. The values
// are formed exactly as the one-block path below forms them. Rows with a nucleus are left alone.
__global__ __launch_bounds__(SPT) void sample_parts_kernel(const float* __restrict__ logits, int vocab, long long row_stride,
                                                           const float* __restrict__ temperature,
                                                           const float* __restrict__ top_p,
                                                           const unsigned* __restrict__ seed,
                                                           const int* __restrict__ counter, Best* __restrict__ parts) {
  __shared__ Best red[SPT / WAVE];
  const int row = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
  const float temp = temperature ? temperature[row] : 0.f;
  const bool sampled = temp > 0.f;
  if (sampled && top_p && top_p[row] < 1.f) return;
  const float* z = logits + (size_t)row * row_stride;
  const int per = (vocab + SPARTS - 1) / SPARTS;
  const int begin = part * per, end = min(vocab, begin + per);
  const float inv_t = sampled ? 1.f / temp : 1.f;
  const uint32_t key = sampled ? mix32(seed[row] ^ mix32((uint32_t)counter[row])) : 0u;
  Best b{-INFINITY, 0x7fffffff};
  for (int i = begin + tid; i < end; i += SPT) {
    float v = z[i];
    if (sampled) v = v * inv_t - logf(-logf(hashed_uniform(key, (uint32_t)i)));
    if (v > b.v) b = Best{v, i};
  }
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    Best o;
    o.v = __shfl_xor(b.v, off, WAVE);
    o.i = __shfl_xor(b.i, off, WAVE);
    b = better(b, o);
  }
  if (tid % WAVE == 0) red[tid / WAVE] = b;
  __syncthreads();
  if (tid == 0) {
#pragma unroll
    for (int w = 1; w < SPT / WAVE; ++w) b = better(b, red[w]);
    parts[(size_t)row * SPARTS + part] = b;
  }
}

// Second kernel, one block per row. temperature / top_p / seed / counter may be null: then every row
// is greedy.
__global__ __launch_bounds__(SNT) void sample_rows_kernel(const float* __restrict__ logits, int vocab, long long row_stride,
                                                          const float* __restrict__ temperature,
                                                          const float* __restrict__ top_p,
                                                          const unsigned* __restrict__ seed,
                                                          const int* __restrict__ counter, const Best* __restrict__ parts,
                                                          int* __restrict__ tokens) {
  __shared__ Best red_b[SNT / WAVE];
  __shared__ float red_f[SNT / WAVE];
  __shared__ int scan[SNT];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (size_t)row * row_stride;
  const float temp = temperature ? temperature[row] : 0.f;
  const float nucleus = (temp > 0.f && top_p) ? top_p[row] : 1.f;

  if (!(nucleus < 1.f)) {  // the first kernel has searched this row
    Best b = tid < SPARTS ? parts[(size_t)row * SPARTS + tid] : Best{-INFINITY, 0x7fffffff};
    b = block_best(b, red_b);
    if (tid == 0) tokens[row] = b.i == 0x7fffffff ? 0 : b.i;
    return;
  }

  const float inv_t = 1.f / temp;
  const uint32_t key = mix32(seed[row] ^ mix32((uint32_t)counter[row]));
  float cut = 0.f;     // tokens with probability > cut stay
  int ties_kept = 0;   // and the first ties_kept tokens with probability == cut
  float zmax = 0.f, inv_sum = 0.f;

  Best top{-INFINITY, 0};
  for (int i = tid; i < vocab; i += SNT) top.v = fmaxf(top.v, z[i] * inv_t);
  zmax = block_best(top, red_b).v;
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

  // Rank of each tie by index needs index order across threads: contiguous chunks per thread.
  const int chunk = (vocab + SNT - 1) / SNT;
  const int begin = tid * chunk, end = min(vocab, begin + chunk);
  int tie_rank = 0;
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

  Best b{-INFINITY, 0x7fffffff};
  for (int i = begin; i < end; ++i) {
    const float zi = z[i] * inv_t;
    const float p = expf(zi - zmax) * inv_sum;
    if (p < cut) continue;
    if (p == cut && tie_rank++ >= ties_kept) continue;
    const float u = hashed_uniform(key, (uint32_t)i);
    const float v = zi - logf(-logf(u));
    if (v > b.v) b = Best{v, i};
  }
  b = block_best(b, red_b);
  if (tid == 0) tokens[row] = b.i == 0x7fffffff ? 0 : b.i;
}

// Bytes of the scratch buffer ms_sample_rows needs for `rows` rows (-1: too many rows).
extern "C" int ms_sample_scratch_bytes(int rows) {
  const long long n = (long long)(rows > 0 ? rows : 0) * SPARTS * (long long)sizeof(Best);
  return n > 0x7fffffffLL ? -1 : (int)n;
}

extern "C" int ms_sample_rows(const float* logits, int rows, int vocab, long long row_stride, const float* temperature,
                              const float* top_p, const unsigned* seed, const int* counter, void* scratch, int* tokens,
                              hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (vocab <= 0 || row_stride < vocab || scratch == nullptr) return MS_BAD_ARG;
  if (temperature != nullptr && (seed == nullptr || counter == nullptr)) return MS_BAD_ARG;
  sample_parts_kernel<<<dim3(rows, SPARTS), SPT, 0, st>>>(logits, vocab, row_stride, temperature, top_p, seed, counter,
                                                         (Best*)scratch);
  sample_rows_kernel<<<rows, SNT, 0, st>>>(logits, vocab, row_stride, temperature, top_p, seed, counter,
                                           (const Best*)scratch, tokens);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// The same two kernels over a scratch buffer that lives in the library instead of in the caller's
// allocation, for callers that cannot allocate (declared in sampling.h).

static __device__ __align__(256) unsigned char sample_static_scratch[MS_SAMPLE_STATIC_MAX_ROWS * SPARTS * sizeof(Best)];

#define MS_MAX_DEVICES 64
static void* sample_static_ptr[MS_MAX_DEVICES];  // per device: where that device's copy of the array lies
static std::mutex sample_static_mutex;

// The device address of the current device's copy of the array, looked up once per device. In host
// code the array's name is only a handle for this lookup; kernels are given the address it returns.
static void* sample_static_scratch_ptr() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MS_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lock(sample_static_mutex);
  if (sample_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(sample_static_scratch)) != hipSuccess) return nullptr;
    sample_static_ptr[dev] = p;
  }
  return sample_static_ptr[dev];
}

extern "C" int ms_sample_rows_static_max_rows() { return MS_SAMPLE_STATIC_MAX_ROWS; }

extern "C" int ms_sample_rows_static(const float* logits, int rows, int vocab, long long row_stride,
                                     const float* temperature, const float* top_p, const unsigned* seed,
                                     const int* counter, int* tokens, hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (rows > MS_SAMPLE_STATIC_MAX_ROWS) return MS_UNSUPPORTED;
  if (vocab <= 0 || row_stride < vocab || logits == nullptr || tokens == nullptr) return MS_BAD_ARG;
  if (temperature != nullptr && (seed == nullptr || counter == nullptr)) return MS_BAD_ARG;
  Best* parts = (Best*)sample_static_scratch_ptr();
  if (parts == nullptr) return MS_LAUNCH_FAILED;
  // Nothing in the array has to start at zero: the first kernel writes every part of every row that the
  // second kernel reads (rows with a nucleus are neither written nor read), whatever an earlier call left.
  sample_parts_kernel<<<dim3(rows, SPARTS), SPT, 0, st>>>(logits, vocab, row_stride, temperature, top_p, seed, counter, parts);
  sample_rows_kernel<<<rows, SNT, 0, st>>>(logits, vocab, row_stride, temperature, top_p, seed, counter, parts, tokens);
  return launch_status();
}
