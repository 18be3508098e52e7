// Causal grouped-query attention over the paged cache, generic form: any head size that is a
// multiple of 16 up to 256, any head counts, float32 or bfloat16 storage, float32 arithmetic.
//
// One wave per (token, query head); ``token_list`` (optional) names the flat token indices to run. Keys are visited in tiles of 64 aligned to absolute positions
// (tile boundaries at multiples of 64), so what a query computes depends only on its position, the
// window and the cache contents: not on how tokens were cut into steps or batched.
//   scores: lane = key; softmax: running maximum and sum (float32); values: lane = head element.
//
// Cache layouts: keys [pages, Hkv, page_size, D], values [pages, Hkv, D, page_size] (transposed
// within the page); block_table[row, i] = page of the row's tokens
// i * page_size .. ; a query at position p of row b sees keys max(0, p - window + 1) .. p
// (window == 0: all keys 0 .. p). Query head h reads KV head h / (Hq / Hkv).
#include "common.h"

#define MAX_HEAD_DIM 256

template <typename T> struct Vec16;  // 16 bytes of T
template <> struct Vec16<float> { static constexpr int N = 4; };
template <> struct Vec16<bf16> { static constexpr int N = 8; };

template <typename T>
__global__ __launch_bounds__(WAVE) void paged_attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ token_list,
    const int* __restrict__ token_row, const int* __restrict__ pos, T* __restrict__ out, int Hq, int Hkv, int D,
    int page_size, float scale, int window) {
  __shared__ __attribute__((aligned(16))) float qs[MAX_HEAD_DIM];
  __shared__ float ps[WAVE];
  constexpr int VN = Vec16<T>::N;
  constexpr int PER = MAX_HEAD_DIM / WAVE;
  const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (Hq / Hkv);
  const int p = pos[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* table = block_table + (size_t)token_row[t] * table_width;

  const T* qv = q + (size_t)t * q_stride + (size_t)h * D;
  for (int e = lane; e < D; e += WAVE) qs[e] = to_f32(qv[e]);
  __syncthreads();

  float m_run = -INFINITY, l_run = 0.f;
  float o[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) o[i] = 0.f;

  for (int j0 = (lo / WAVE) * WAVE; j0 <= p; j0 += WAVE) {
    const int j = j0 + lane;
    const bool valid = j >= lo && j <= p;
    float s = -INFINITY;
    if (valid) {
      const int page = table[j / page_size];
      const T* kp = kc + (((size_t)page * Hkv + kvh) * page_size + (j % page_size)) * D;
      float dot = 0.f;
      for (int d = 0; d < D; d += VN) {
        alignas(16) T kv[VN];
        *reinterpret_cast<uint4*>(kv) = *reinterpret_cast<const uint4*>(kp + d);
#pragma unroll
        for (int i = 0; i < VN; ++i) dot = fmaf(qs[d + i], to_f32(kv[i]), dot);
      }
      s = dot * scale;
    }
    const float m_new = fmaxf(m_run, wave_max(s));  // finite: every visited tile holds a visible key
    const float pj = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m_run - m_new);
    l_run = l_run * corr + wave_sum(pj);
    m_run = m_new;
    __syncthreads();
    ps[lane] = pj;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PER; ++i) o[i] *= corr;
    const int jb = j0 > lo ? j0 : lo;
    const int je = j0 + WAVE - 1 < p ? j0 + WAVE - 1 : p;
    for (int jj = jb; jj <= je; ++jj) {
      const int page = table[jj / page_size];
      const T* vp = vc + ((size_t)page * Hkv + kvh) * D * page_size + (jj % page_size);
      const float w = ps[jj - j0];
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int e = lane + i * WAVE;
        if (e < D) o[i] = fmaf(w, to_f32(vp[(size_t)e * page_size]), o[i]);
      }
    }
  }
  T* ov = out + ((size_t)t * Hq + h) * D;
  const float inv = 1.f / l_run;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + i * WAVE;
    if (e < D) ov[e] = from_f32<T>(o[i] * inv);
  }
}

extern "C" int ms_paged_attention_generic(const void* q, int q_stride, const void* kc, const void* vc, int is_bf16,
                                          const int* block_table, int table_width, const int* token_list,
                                          const int* token_row, const int* pos, void* out, int tokens, int Hq, int Hkv,
                                          int D, int page_size, float scale, int window, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (D <= 0 || D > MAX_HEAD_DIM || D % 16 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || page_size <= 0 || window < 0 ||
      table_width <= 0 || Hq > 65535 || q_stride < Hq * D)
    return MS_BAD_ARG;
  dim3 grid(tokens, Hq);
  if (is_bf16)
    paged_attention_generic_kernel<bf16><<<grid, WAVE, 0, st>>>((const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc,
                                                                block_table, table_width, token_list, token_row, pos,
                                                                (bf16*)out, Hq, Hkv, D, page_size, scale, window);
  else
    paged_attention_generic_kernel<float><<<grid, WAVE, 0, st>>>((const float*)q, q_stride, (const float*)kc,
                                                                 (const float*)vc, block_table, table_width, token_list,
                                                                 token_row, pos, (float*)out, Hq, Hkv, D, page_size, scale,
                                                                 window);
  return launch_status();
}
