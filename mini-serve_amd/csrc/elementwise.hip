// Embedding gather, RMSNorm, gated activation, casts, and the fused per-head norm + rotation +
// cache store. All arithmetic is float32; bfloat16 appears only as a storage type and each
// result is rounded once.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// out[t, :] = float(table[ids[t], :])
template <typename TW>
__global__ void embed_kernel(const int* __restrict__ ids, const TW* __restrict__ table, float* __restrict__ out, int width) {
  const int t = blockIdx.x;
  const TW* src = table + (size_t)ids[t] * width;
  float* dst = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_f32(src[i]);
}

extern "C" int ms_embed(const int* ids, const void* table, int table_is_bf16, float* out, int tokens, int width, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (width <= 0) return MS_BAD_ARG;
  if (table_is_bf16)
    embed_kernel<bf16><<<tokens, 256, 0, st>>>(ids, (const bf16*)table, out, width);
  else
    embed_kernel<float><<<tokens, 256, 0, st>>>(ids, (const float*)table, out, width);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// y[r, :] = w * x[row(r), :] * rsqrt(mean(x^2) + eps), float32 throughout, rounded once.
// With `parts` (float [splits, rows_total, width], the partial sums of a matrix product that still
// has to be added to the residual stream) the row is first brought up to date: x[row] + sum over
// splits in ascending order. Without a row list x is updated in place; with one x is left unchanged
// (a list may name a row twice).
// One block of NT threads per row; each thread keeps up to KEEP of its elements in registers between
// the two passes (wider rows are read again). Few rows (a decode step) run with 1024 threads so that
// all loads of a row are in flight at once.
template <typename TW, typename TO, int NT, int KEEP>
__global__ __launch_bounds__(NT) void rmsnorm_kernel(float* __restrict__ x, const TW* __restrict__ w, TO* __restrict__ y,
                                                     const int* __restrict__ rows, int width, float eps,
                                                     const float* __restrict__ parts, int splits, size_t split_stride) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x;
  const size_t row = rows ? rows[r] : r;
  float* src = x + row * width;
  const bool in_place = parts != nullptr && rows == nullptr;
  float kept[KEEP];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int i = threadIdx.x + j * NT;
    float v = 0.f;
    if (i < width) {
      v = src[i];
      if (parts != nullptr) {
        v += sum_splits(parts + row * width + i, splits, split_stride);
        if (in_place) src[i] = v;
      }
    }
    kept[j] = v;
    ss += v * v;
  }
  for (int i = threadIdx.x + KEEP * NT; i < width; i += NT) {  // rows wider than NT * KEEP
    float v = src[i];
    if (parts != nullptr) {
      v += sum_splits(parts + row * width + i, splits, split_stride);
      if (in_place) src[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float rstd = rsqrtf(ss / (float)width + eps);
  TO* dst = y + (size_t)r * width;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int i = threadIdx.x + j * NT;
    if (i < width) dst[i] = from_f32<TO>(kept[j] * rstd * to_f32(w[i]));
  }
  for (int i = threadIdx.x + KEEP * NT; i < width; i += NT) {
    float v = src[i];  // in place: this thread's own update; otherwise the sum is formed again
    if (parts != nullptr && !in_place) v += sum_splits(parts + row * width + i, splits, split_stride);
    dst[i] = from_f32<TO>(v * rstd * to_f32(w[i]));
  }
}

extern "C" int ms_rmsnorm(float* x, const void* w, int w_is_bf16, void* y, int y_is_bf16, const int* rows, int n_rows,
                          int width, float eps, const float* parts, int splits, long long split_stride, hipStream_t st) {
  if (n_rows <= 0) return MS_OK;
  if (width <= 0 || (parts != nullptr && splits < 1)) return MS_BAD_ARG;
  // float32 output keeps one block shape for every batch, so that its sums are formed in one order
  // whatever the batch; bfloat16 output takes the wide block for few rows.
  const bool wide = y_is_bf16 && n_rows <= 256;
#define LAUNCH(TW, TO)                                                                                                  \
  if (wide)                                                                                                             \
    rmsnorm_kernel<TW, TO, 1024, 4><<<n_rows, 1024, 0, st>>>(x, (const TW*)w, (TO*)y, rows, width, eps, parts, splits,  \
                                                              (size_t)split_stride);                                    \
  else                                                                                                                  \
    rmsnorm_kernel<TW, TO, 256, 8><<<n_rows, 256, 0, st>>>(x, (const TW*)w, (TO*)y, rows, width, eps, parts, splits,    \
                                                            (size_t)split_stride)
  if (w_is_bf16 && y_is_bf16) { LAUNCH(bf16, bf16); }
  else if (w_is_bf16) { LAUNCH(bf16, float); }
  else if (y_is_bf16) { LAUNCH(float, bf16); }
  else { LAUNCH(float, float); }
#undef LAUNCH
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i]
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const float g = to_f32(gu[(size_t)t * 2 * inter + i]);
  const float u = to_f32(gu[(size_t)t * 2 * inter + inter + i]);
  out[(size_t)t * inter + i] = from_f32<T>(g / (1.f + expf(-g)) * u);
}

// The same with gu given as float partial sums [splits, tokens, 2 * inter] (summed in ascending order).
template <typename T>
__global__ void silu_mul_parts_kernel(const float* __restrict__ parts, int splits, size_t split_stride,
                                      T* __restrict__ out, int inter) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const float* row = parts + (size_t)t * 2 * inter;
  const float g = sum_splits(row + i, splits, split_stride);
  const float u = sum_splits(row + inter + i, splits, split_stride);
  out[(size_t)t * inter + i] = from_f32<T>(g / (1.f + expf(-g)) * u);
}

extern "C" int ms_silu_mul(const void* gu, void* out, int is_bf16, int tokens, int inter, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (inter <= 0 || tokens > 65535) return MS_BAD_ARG;
  dim3 grid((inter + 255) / 256, tokens);
  if (is_bf16) silu_mul_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)gu, (bf16*)out, inter);
  else silu_mul_kernel<float><<<grid, 256, 0, st>>>((const float*)gu, (float*)out, inter);
  return launch_status();
}

extern "C" int ms_silu_mul_parts(const float* parts, int splits, long long split_stride, void* out, int out_is_bf16,
                                 int tokens, int inter, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (inter <= 0 || tokens > 65535 || splits < 1) return MS_BAD_ARG;
  dim3 grid((inter + 255) / 256, tokens);
  if (out_is_bf16) silu_mul_parts_kernel<bf16><<<grid, 256, 0, st>>>(parts, splits, (size_t)split_stride, (bf16*)out, inter);
  else silu_mul_parts_kernel<float><<<grid, 256, 0, st>>>(parts, splits, (size_t)split_stride, (float*)out, inter);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<TO>(to_f32(in[i]));
}

extern "C" int ms_cast(const void* in, int in_is_bf16, void* out, int out_is_bf16, long long n, hipStream_t st) {
  if (n <= 0) return MS_OK;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (in_is_bf16 && !out_is_bf16) cast_kernel<bf16, float><<<blocks, 256, 0, st>>>((const bf16*)in, (float*)out, (size_t)n);
  else if (!in_is_bf16 && out_is_bf16) cast_kernel<float, bf16><<<blocks, 256, 0, st>>>((const float*)in, (bf16*)out, (size_t)n);
  else return MS_BAD_ARG;
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// One block of 4 waves per (token, four head slots): a wave per head slot. Head slots [0, Hq)
// are query heads, [Hq, Hq+Hkv) key heads, [Hq+Hkv, Hq+2Hkv) value heads of the token's row in
// qkv [tokens, (Hq + 2 Hkv) * D].
//   q, k: optional RMSNorm over the head (weight [D]), then rotation of the first `rot` elements in
//         pairs (j, j + rot/2) by angle float(pos) * inv_freq[j] (sine and cosine are formed once per
//         block and shared by its four heads);
//   q goes to q_out; k and v go to the cache page of the token's slot
//   (slot = page * page_size + offset; keys [pages, Hkv, page_size, D], values transposed within
//   the page, [pages, Hkv, D, page_size]).
// With slots == nullptr only the query heads are processed (the entry reads another entry's cache).
#define MAX_HEAD_DIM 256
template <typename T, typename TW>
__global__ __launch_bounds__(256) void qk_norm_rope_store_kernel(
    const T* qkv, const float* __restrict__ parts, int splits, size_t split_stride, T* q_out, int q_out_stride,
    const int* __restrict__ pos, const int* __restrict__ slots, const TW* __restrict__ qw, const TW* __restrict__ kw,
    float eps, const float* __restrict__ inv_freq, int rot, T* __restrict__ kc, T* __restrict__ vc, int Hq, int Hkv, int D,
    int page_size, int heads) {
  __shared__ float cs[MAX_HEAD_DIM / 2], sn[MAX_HEAD_DIM / 2];
  __shared__ float buf[4][MAX_HEAD_DIM];
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int hs = blockIdx.y * 4 + wave;  // this wave's head slot
  const int half = rot / 2;
  if (threadIdx.x < half) {
    float s, c;
    sincosf((float)pos[t] * inv_freq[threadIdx.x], &s, &c);
    cs[threadIdx.x] = c;
    sn[threadIdx.x] = s;
  }
  __syncthreads();
  constexpr int PER = MAX_HEAD_DIM / WAVE;
  if (hs < heads) {
    const int kind = hs < Hq ? 0 : (hs < Hq + Hkv ? 1 : 2);
    const size_t at = ((size_t)t * (Hq + 2 * Hkv) + hs) * D;
    float x[PER];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane + i * WAVE;
      float v = 0.f;
      if (e < D) {
        if (parts != nullptr) {
          v = sum_splits(parts + at + e, splits, split_stride);
        } else {
          v = to_f32(qkv[at + e]);
        }
      }
      x[i] = v;
      ss += v * v;
    }
    T* dst = q_out + (size_t)t * q_out_stride + (size_t)hs * D;  // for a query head
    size_t dst_step = 1;  // distance between consecutive head elements at the destination
    if (kind == 1) {
      const int s = slots[t];
      dst = kc + (((size_t)(s / page_size) * Hkv + (hs - Hq)) * page_size + (s % page_size)) * D;
    } else if (kind == 2) {
      const int s = slots[t];
      dst = vc + ((size_t)(s / page_size) * Hkv + (hs - Hq - Hkv)) * D * page_size + (s % page_size);
      dst_step = page_size;
    }
    if (kind != 2) {
      const TW* w = kind == 0 ? qw : kw;
      if (w != nullptr) {
        ss = wave_sum(ss);
        const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int e = lane + i * WAVE;
          if (e < D) x[i] = x[i] * rstd * to_f32(w[e]);
        }
      }
      if (rot > 0) {
        // The wave exchanges the partners of its pairs through its own LDS row; a wave runs in
        // lockstep, so no block barrier is needed between its write and its read.
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int e = lane + i * WAVE;
          if (e < D) buf[wave][e] = x[i];
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int e = lane + i * WAVE;
          if (e < rot) {
            const int j = e < half ? e : e - half;
            x[i] = e < half ? x[i] * cs[j] - buf[wave][e + half] * sn[j] : x[i] * cs[j] + buf[wave][e - half] * sn[j];
          }
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane + i * WAVE;
      if (e < D) dst[(size_t)e * dst_step] = from_f32<T>(x[i]);
    }
  }
}

// Source: qkv [tokens, (Hq + 2 Hkv) D], or (parts != nullptr) float partial sums [splits, tokens, (Hq + 2 Hkv) D] of it.
// Queries go to q_out [tokens, q_out_stride >= Hq D] (which may be qkv itself: in place).
extern "C" int ms_qk_norm_rope_store(const void* qkv, const float* parts, int splits, long long split_stride, void* q_out,
                                     int q_out_stride, int is_bf16, const int* pos, const int* slots, const void* qw,
                                     const void* kw, int w_is_bf16, float eps, const float* inv_freq, int rot, void* kc,
                                     void* vc, int tokens, int Hq, int Hkv, int D, int page_size, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if ((qkv == nullptr) == (parts == nullptr) || (parts != nullptr && splits < 1) || q_out == nullptr || q_out_stride < Hq * D)
    return MS_BAD_ARG;
  if (D <= 0 || D > MAX_HEAD_DIM || rot < 0 || rot > D || (rot & 1) || Hq <= 0 || Hkv <= 0 || page_size <= 0) return MS_BAD_ARG;
  if ((qw == nullptr) != (kw == nullptr)) return MS_BAD_ARG;
  if (rot > 0 && inv_freq == nullptr) return MS_BAD_ARG;
  const int heads = slots ? Hq + 2 * Hkv : Hq;
  if ((heads + 3) / 4 > 65535) return MS_BAD_ARG;
#define LAUNCH(T, TW)                                                                                                   \
  qk_norm_rope_store_kernel<T, TW><<<dim3(tokens, (heads + 3) / 4), 256, 0, st>>>((const T*)qkv, parts, splits, (size_t)split_stride, (T*)q_out, \
                                                            q_out_stride, pos, slots, (const TW*)qw, (const TW*)kw, eps,  \
                                                            inv_freq, rot, (T*)kc, (T*)vc, Hq, Hkv, D, page_size, heads)
  if (is_bf16 && w_is_bf16) LAUNCH(bf16, bf16);
  else if (is_bf16) LAUNCH(bf16, float);
  else if (w_is_bf16) LAUNCH(float, bf16);
  else LAUNCH(float, float);
#undef LAUNCH
  return launch_status();
}
