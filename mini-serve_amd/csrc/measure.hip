// Kernels that measure what the memory system gives: a streaming read (every 16-byte vector of a
// buffer is loaded once and folded into a sum that is kept so that the loads stay) and a streaming
// copy. They are the denominators beside which the decode step's bytes per second are read; the model
// never calls them.
#include "common.h"

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// The blocks take chunks of 256 * U vectors in turn (block b the chunks b, b + blocks, ...), so that at
// any time the chip reads one contiguous window of the buffer; a thread has U loads in flight. Block b
// leaves the xor of what it saw in out[b].
constexpr int READ_U = 8, COPY_U = 4;

__global__ __launch_bounds__(256) void read_stream_kernel(const u32x4* __restrict__ p, size_t vectors, unsigned* __restrict__ out) {
  constexpr size_t chunk = 256 * READ_U;
  u32x4 acc = {0u, 0u, 0u, 0u};
  size_t base = (size_t)blockIdx.x * chunk;
  for (; base + chunk <= vectors; base += (size_t)gridDim.x * chunk) {
    u32x4 v[READ_U];
#pragma unroll
    for (int u = 0; u < READ_U; ++u) v[u] = __builtin_nontemporal_load(&p[base + u * 256 + threadIdx.x]);
#pragma unroll
    for (int u = 0; u < READ_U; ++u) acc ^= v[u];
  }
  for (size_t i = base + threadIdx.x; i < vectors && i < base + chunk; i += 256) acc ^= p[i];  // the last, partial chunk
  unsigned x = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) x ^= __shfl_xor(x, off, WAVE);
  __shared__ unsigned red[4];
  if (threadIdx.x % WAVE == 0) red[threadIdx.x / WAVE] = x;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = red[0] ^ red[1] ^ red[2] ^ red[3];
}

__global__ __launch_bounds__(256) void copy_stream_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t vectors) {
  constexpr size_t chunk = 256 * COPY_U;
  size_t base = (size_t)blockIdx.x * chunk;
  for (; base + chunk <= vectors; base += (size_t)gridDim.x * chunk) {
    u32x4 v[COPY_U];
#pragma unroll
    for (int u = 0; u < COPY_U; ++u) v[u] = __builtin_nontemporal_load(&src[base + u * 256 + threadIdx.x]);
#pragma unroll
    for (int u = 0; u < COPY_U; ++u) __builtin_nontemporal_store(v[u], &dst[base + u * 256 + threadIdx.x]);
  }
  for (size_t i = base + threadIdx.x; i < vectors && i < base + chunk; i += 256) dst[i] = src[i];
}

// Reads `bytes` (a multiple of 16, 16-byte aligned) with `blocks` blocks; out holds `blocks` words.
extern "C" int ms_measure_read(const void* p, long long bytes, int blocks, unsigned* out, hipStream_t st) {
  if (bytes <= 0 || bytes % 16 || blocks < 1 || blocks > 65535 * 16 || p == nullptr || out == nullptr) return MS_BAD_ARG;
  read_stream_kernel<<<(unsigned)blocks, 256, 0, st>>>((const u32x4*)p, (size_t)(bytes / 16), out);
  return launch_status();
}

// Copies `bytes` (a multiple of 16, both 16-byte aligned, not overlapping) with `blocks` blocks.
extern "C" int ms_measure_copy(const void* src, void* dst, long long bytes, int blocks, hipStream_t st) {
  if (bytes <= 0 || bytes % 16 || blocks < 1 || blocks > 65535 * 16 || src == nullptr || dst == nullptr) return MS_BAD_ARG;
  copy_stream_kernel<<<(unsigned)blocks, 256, 0, st>>>((const u32x4*)src, (u32x4*)dst, (size_t)(bytes / 16));
  return launch_status();
}
