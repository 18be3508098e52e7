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
// Token ids that are still on the device: the last token of row i becomes src[feed[i]] where
// feed[i] >= 0 (a token an earlier step sampled and the host has not read back yet). row_start holds
// rows + 1 offsets into ids; nullptr: every row is one token.
__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ row_start, const int* __restrict__ feed,
                                   const int* __restrict__ src, int rows, int src_len) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows) return;
  const int f = feed[i];
  if (f < 0 || f >= src_len) return;
  ids[row_start ? row_start[i + 1] - 1 : i] = src[f];
}

extern "C" int ms_feed_tokens(int* ids, const int* row_start, const int* feed, const int* src, int rows, int src_len, hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (ids == nullptr || feed == nullptr || src == nullptr || src_len <= 0) return MS_BAD_ARG;
  feed_tokens_kernel<<<(rows + 255) / 256, 256, 0, st>>>(ids, row_start, feed, src, rows, src_len);
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

// The same for few rows of a width that is a multiple of 4 and at most 8 NT, bfloat16 output: NT
// threads per row, a thread owns up to two groups of 4 consecutive elements and moves them as vectors;
// the partial sums of up to 16 splits are fetched at a time. Sums per element in ascending split order, as
// in the kernel above.
// acc += parts of splits s0 .. s0 + B - 1 (those below `splits`), four floats each, in ascending order;
// the B loads are issued before the first sum.
template <int B>
__device__ __forceinline__ void add_splits(float4& acc, const float* __restrict__ p, int s0, int splits, size_t split_stride) {
  float4 t[B];
#pragma unroll
  for (int u = 0; u < B; ++u) {
    const bool in = s0 + u < splits;
    t[u] = *reinterpret_cast<const float4*>(p + (size_t)(in ? s0 + u : 0) * split_stride);
    if (!in) t[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int u = 0; u < B; ++u) {
    acc.x += t[u].x; acc.y += t[u].y; acc.z += t[u].z; acc.w += t[u].w;
  }
}

// Four consecutive weights in one load (w + i is aligned to four elements), kept as loaded: what uses
// them comes after the block's sum, and a conversion right after the load would wait for it there.
template <typename TW> struct Weights4;
template <> struct Weights4<float> {
  float4 v;
  __device__ __forceinline__ void load(const float* w) { v = *reinterpret_cast<const float4*>(w); }
  __device__ __forceinline__ float at(int e) const { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }
};
template <> struct Weights4<bf16> {
  union { uint2 u; bf16 e[4]; } v;
  __device__ __forceinline__ void load(const bf16* w) { v.u = *reinterpret_cast<const uint2*>(w); }
  __device__ __forceinline__ float at(int e) const { return to_f32(v.e[e]); }
};

template <typename TW, int NT>
__global__ __launch_bounds__(NT) void rmsnorm_vec4_kernel(float* __restrict__ x, const TW* __restrict__ w,
                                                            bf16* __restrict__ y, const int* __restrict__ rows, int width,
                                                            float eps, const float* __restrict__ parts, int splits,
                                                            size_t split_stride) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x;
  const size_t row = rows ? rows[r] : r;
  float* src = x + row * width;
  const bool in_place = parts != nullptr && rows == nullptr;
  float4 kept[2];
  Weights4<TW> wk[2];  // asked for with the row: after the block's sum they would cost a second wait
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int i = (threadIdx.x + j * NT) * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < width) {
      wk[j].load(w + i);
      v = *reinterpret_cast<const float4*>(src + i);
      if (parts != nullptr) {
        const float* p = parts + row * width + i;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        // The loads of a batch of splits go out together; few splits (a tile product's two to four) take
        // a batch of their own size, so that no load is issued for nothing. Ascending split order always.
        if (splits <= 2) {
          add_splits<2>(acc, p, 0, splits, split_stride);
        } else if (splits <= 4) {
          add_splits<4>(acc, p, 0, splits, split_stride);
        } else if (splits <= 8) {
          add_splits<8>(acc, p, 0, splits, split_stride);
        } else {  // the products of a decode step leave 12 to 16: one round trip, not two
          for (int s0 = 0; s0 < splits; s0 += 16) add_splits<16>(acc, p, s0, splits, split_stride);
        }
        v.x += acc.x; v.y += acc.y; v.z += acc.z; v.w += acc.w;
        if (in_place) *reinterpret_cast<float4*>(src + i) = v;
      }
    }
    kept[j] = v;
    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
  }
  ss = block_sum<NT>(ss, red);
  const float rstd = rsqrtf(ss / (float)width + eps);
  bf16* dst = y + (size_t)r * width;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int i = (threadIdx.x + j * NT) * 4;
    if (i < width) {
      union { uint2 u; bf16 e[4]; } o;
      o.e[0] = from_f32<bf16>(kept[j].x * rstd * wk[j].at(0));
      o.e[1] = from_f32<bf16>(kept[j].y * rstd * wk[j].at(1));
      o.e[2] = from_f32<bf16>(kept[j].z * rstd * wk[j].at(2));
      o.e[3] = from_f32<bf16>(kept[j].w * rstd * wk[j].at(3));
      *reinterpret_cast<uint2*>(dst + i) = o.u;
    }
  }
}

extern "C" int ms_rmsnorm(float* x, const void* w, int w_is_bf16, void* y, int y_is_bf16, const int* rows, int n_rows,
                          int width, float eps, const float* parts, int splits, long long split_stride, hipStream_t st) {
  if (n_rows <= 0) return MS_OK;
  if (width <= 0 || (parts != nullptr && splits < 1)) return MS_BAD_ARG;
  // float32 output keeps one block shape for every batch, so that its sums are formed in one order
  // whatever the batch; bfloat16 output takes the wide block for few rows.
  const bool wide = y_is_bf16 && n_rows <= 256;
  if (y_is_bf16 && width % 4 == 0 && width <= 8192 && (parts == nullptr || split_stride % 4 == 0)) {
#define LAUNCH_VEC(TW)                                                                                                  \
  if (width <= 2048)                                                                                                    \
    rmsnorm_vec4_kernel<TW, 256><<<n_rows, 256, 0, st>>>(x, (const TW*)w, (bf16*)y, rows, width, eps, parts, splits,    \
                                                          (size_t)split_stride);                                        \
  else                                                                                                                  \
    rmsnorm_vec4_kernel<TW, 1024><<<n_rows, 1024, 0, st>>>(x, (const TW*)w, (bf16*)y, rows, width, eps, parts, splits,  \
                                                            (size_t)split_stride)
    if (w_is_bf16) { LAUNCH_VEC(bf16); } else { LAUNCH_VEC(float); }
#undef LAUNCH_VEC
    return launch_status();
  }
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
// out[t, i] = act(gate[t, i]) * up[t, i] (act: an MS_ACT_* number) for a row gu[t] that holds both, in one of two layouts:
//   block == 0: the gates, then the ups:                 gate i at i, up i at inter + i
//   block  > 0: alternating runs of `block` gates and `block` ups (the order a matrix product over
//               interleaved weight rows leaves them in): gate i at (i / block) * 2 block + i % block,
//               up i `block` further on. inter is a multiple of block then.
__device__ __forceinline__ int gate_at(int i, int block) { return block ? (i / block) * 2 * block + i % block : i; }
__device__ __forceinline__ int up_at(int i, int inter, int block) { return block ? gate_at(i, block) + block : inter + i; }

template <typename T>
__global__ void act_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int block, int act) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const float g = to_f32(gu[(size_t)t * 2 * inter + gate_at(i, block)]);
  const float u = to_f32(gu[(size_t)t * 2 * inter + up_at(i, inter, block)]);
  out[(size_t)t * inter + i] = from_f32<T>(activate(g, act) * u);
}

// The same with gu given as float partial sums [splits, tokens, 2 * inter] (summed in ascending order).
template <typename T>
__global__ void act_mul_parts_kernel(const float* __restrict__ parts, int splits, size_t split_stride,
                                     T* __restrict__ out, int inter, int block, int act) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const float* row = parts + (size_t)t * 2 * inter;
  const float g = sum_splits(row + gate_at(i, block), splits, split_stride);
  const float u = sum_splits(row + up_at(i, inter, block), splits, split_stride);
  out[(size_t)t * inter + i] = from_f32<T>(activate(g, act) * u);
}

// bfloat16 with inter (and block) a multiple of 8: eight elements per thread, moved as 16-byte vectors.
__global__ void act_mul_vec8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int inter, int block, int act) {
  const int t = blockIdx.y;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= inter) return;
  union V { uint4 u; bf16 e[8]; } g, u, o;
  g.u = *reinterpret_cast<const uint4*>(gu + (size_t)t * 2 * inter + gate_at(i, block));
  u.u = *reinterpret_cast<const uint4*>(gu + (size_t)t * 2 * inter + up_at(i, inter, block));
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float gv = to_f32(g.e[e]);
    o.e[e] = from_f32<bf16>(activate(gv, act) * to_f32(u.e[e]));
  }
  *reinterpret_cast<uint4*>(out + (size_t)t * inter + i) = o.u;
}

extern "C" int ms_act_mul(const void* gu, void* out, int is_bf16, int tokens, int inter, int block, int act, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (inter <= 0 || tokens > 65535 || block < 0 || (block > 0 && inter % block) || act < 0 || act >= MS_ACT_COUNT) return MS_BAD_ARG;
  dim3 grid((inter + 255) / 256, tokens);
  if (is_bf16 && inter % 8 == 0 && block % 8 == 0)
    act_mul_vec8_kernel<<<dim3((inter / 8 + 255) / 256, tokens), 256, 0, st>>>((const bf16*)gu, (bf16*)out, inter, block, act);
  else if (is_bf16) act_mul_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)gu, (bf16*)out, inter, block, act);
  else act_mul_kernel<float><<<grid, 256, 0, st>>>((const float*)gu, (float*)out, inter, block, act);
  return launch_status();
}

extern "C" int ms_act_mul_parts(const float* parts, int splits, long long split_stride, void* out, int out_is_bf16,
                                int tokens, int inter, int block, int act, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (inter <= 0 || tokens > 65535 || splits < 1 || block < 0 || (block > 0 && inter % block) || act < 0 || act >= MS_ACT_COUNT)
    return MS_BAD_ARG;
  dim3 grid((inter + 255) / 256, tokens);
  if (out_is_bf16) act_mul_parts_kernel<bf16><<<grid, 256, 0, st>>>(parts, splits, (size_t)split_stride, (bf16*)out, inter, block, act);
  else act_mul_parts_kernel<float><<<grid, 256, 0, st>>>(parts, splits, (size_t)split_stride, (float*)out, inter, block, act);
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
// Cosines and sines of a step's rotation angles, table [tokens, 2 * half]: cos(a) in the first half of
// a row, sin(a) in the second, a = float(pos[t]) * inv_freq[j]. Made once per step and read by every
// layer's rotation kernel.
__global__ void rope_table_kernel(const int* __restrict__ pos, const float* __restrict__ inv_freq, float* __restrict__ out,
                                  int tokens, int half) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= tokens * half) return;
  const int t = i / half, j = i % half;
  float sn, cs;
  sincosf((float)pos[t] * inv_freq[j], &sn, &cs);
  out[(size_t)t * 2 * half + j] = cs;
  out[(size_t)t * 2 * half + half + j] = sn;
}

extern "C" int ms_rope_table(const int* pos, const float* inv_freq, float* out, int tokens, int half, hipStream_t st) {
  if (tokens <= 0 || half <= 0) return MS_OK;
  if ((long long)tokens * half > 0x7fffffffLL) return MS_BAD_ARG;
  rope_table_kernel<<<(tokens * half + 255) / 256, 256, 0, st>>>(pos, inv_freq, out, tokens, half);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Head slots [0, Hq) are query heads, [Hq, Hq+Hkv) key heads, [Hq+Hkv, Hq+2Hkv) value heads of the
// token's row in qkv [tokens, (Hq + 2 Hkv) * D].
//   q, k: optional RMSNorm over the head (weight [D]), then rotation of the first `rot` elements in
//         pairs by the angle whose cosine and sine are rope[t][j] and rope[t][rot/2 + j] for pair j: the
//         elements (j, j + rot/2) (MS_ROPE_HALVES) or (2j, 2j + 1) (MS_ROPE_ADJACENT);
//   q goes to q_out; k and v go to the cache page of the token's slot
//   (slot = page * page_size + offset; keys [pages, Hkv, page_size, D], values transposed within
//   the page, [pages, Hkv, D, page_size]).
// With slots == nullptr only the query heads are processed (the entry reads another entry's cache).
//
// General kernel (any head size up to 256, rotation over part of the head): one block of 4 waves per
// (token, four head slots), a wave per head slot.
#define MAX_HEAD_DIM 256
template <typename T, typename TW>
__global__ __launch_bounds__(256) void qk_norm_rope_store_kernel(
    const T* qkv, const float* __restrict__ parts, int splits, size_t split_stride, T* q_out, int q_out_stride,
    const int* __restrict__ slots, const TW* __restrict__ qw, const TW* __restrict__ kw, float eps,
    const float* __restrict__ rope, int rot, int pairing, T* __restrict__ kc, T* __restrict__ vc, int Hq, int Hkv, int D,
    int page_size, int heads) {
  __shared__ float buf[4][MAX_HEAD_DIM];
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int hs = blockIdx.y * 4 + wave;  // this wave's head slot
  const int half = rot / 2;
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
        const float* cs = rope + (size_t)t * rot;
        const float* sn = cs + half;
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
            // first of its pair: x cos - partner sin; second: x cos + partner sin
            const bool first = pairing == MS_ROPE_ADJACENT ? (e & 1) == 0 : e < half;
            const int j = pairing == MS_ROPE_ADJACENT ? e / 2 : (e < half ? e : e - half);
            const int partner = pairing == MS_ROPE_ADJACENT ? (e ^ 1) : (e < half ? e + half : e - half);
            x[i] = first ? x[i] * cs[j] - buf[wave][partner] * sn[j] : x[i] * cs[j] + buf[wave][partner] * sn[j];
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

// D = 64 or 128, rotation over the whole head or none: one block per
// (256 / (D/8) consecutive tokens, head slot). A thread owns 8 consecutive elements of one token's
// head, moved as one vector; the D/8 threads of a token are neighbours in a wave and share the sum of
// squares and the rotation partners (thread i and thread i ^ D/16) through lane exchanges. Value
// heads are turned in LDS so that a thread writes 8 consecutive tokens of one head element with one
// vector store where those tokens fill an aligned run of a page (single stores otherwise).
template <typename T>
struct Vec8;
template <>
struct Vec8<bf16> {
  uint4 raw;
  __device__ __forceinline__ void load(const bf16* p) { raw = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void store(bf16* p) const { *reinterpret_cast<uint4*>(p) = raw; }
  __device__ __forceinline__ float get(int i) const { return to_f32(reinterpret_cast<const bf16*>(&raw)[i]); }
  __device__ __forceinline__ void set(int i, float v) { reinterpret_cast<bf16*>(&raw)[i] = from_f32<bf16>(v); }
};
template <>
struct Vec8<float> {
  float4 lo, hi;
  __device__ __forceinline__ void load(const float* p) {
    lo = *reinterpret_cast<const float4*>(p);
    hi = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ __forceinline__ void store(float* p) const {
    *reinterpret_cast<float4*>(p) = lo;
    *reinterpret_cast<float4*>(p + 4) = hi;
  }
  __device__ __forceinline__ float get(int i) const { return i < 4 ? (&lo.x)[i] : (&hi.x)[i - 4]; }
  __device__ __forceinline__ void set(int i, float v) {
    if (i < 4) (&lo.x)[i] = v;
    else (&hi.x)[i - 4] = v;
  }
};

template <typename T, typename TW, int D, int HPB>
__global__ __launch_bounds__(256) void qk_norm_rope_store_tile_kernel(
    const T* qkv, const float* __restrict__ parts, int splits, size_t split_stride, T* q_out, int q_out_stride,
    const int* __restrict__ slots, const TW* __restrict__ qw, const TW* __restrict__ kw, float eps,
    const float* __restrict__ rope, T* __restrict__ kc, T* __restrict__ vc, int tokens, int Hq, int Hkv, int page_size) {
  constexpr int TPT = D / 8;      // threads per token
  constexpr int TOK = 256 / TPT;  // tokens per block
  constexpr int RUNS = TOK / 8;   // runs of 8 tokens
  __shared__ __attribute__((aligned(16))) T vt[TOK][D + 8];
  // blockIdx.y walks groups of up to HPB heads of one kind: query groups, then key groups, then value
  // groups. A thread loads its 8 elements of every head of the group before it works on any (HPB
  // loads in flight), and the rotation's cosines and sines once for all of them.
  const int nq = (Hq + HPB - 1) / HPB, nk = (Hkv + HPB - 1) / HPB;
  int kind, h0, of_kind;
  if ((int)blockIdx.y < nq) { kind = 0; h0 = blockIdx.y * HPB; of_kind = Hq; }
  else if ((int)blockIdx.y < nq + nk) { kind = 1; h0 = (blockIdx.y - nq) * HPB; of_kind = Hkv; }
  else { kind = 2; h0 = (blockIdx.y - nq - nk) * HPB; of_kind = Hkv; }
  const int hn = min(HPB, of_kind - h0);                           // heads of this block
  const int hs0 = (kind == 0 ? 0 : (kind == 1 ? Hq : Hq + Hkv)) + h0;  // its first head slot
  const int tl = threadIdx.x / TPT, i = threadIdx.x % TPT;
  const int t0 = blockIdx.x * TOK, t = t0 + tl;
  const bool live = t < tokens;
  const size_t at0 = ((size_t)(live ? t : tokens - 1) * (Hq + 2 * Hkv) + hs0) * D + i * 8;

  float x[HPB][8];
#pragma unroll
  for (int h = 0; h < HPB; ++h) {
    const size_t at = at0 + (size_t)(h < hn ? h : 0) * D;
    if (parts != nullptr) {
#pragma unroll
      for (int e = 0; e < 8; ++e) x[h][e] = 0.f;
      for (int s0 = 0; s0 < splits; s0 += 4) {  // ascending split order; the loads of four splits go out together
        float4 a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bool in = s0 + u < splits;
          const float* src = parts + (size_t)(in ? s0 + u : 0) * split_stride + at;
          a[u] = *reinterpret_cast<const float4*>(src);
          b[u] = *reinterpret_cast<const float4*>(src + 4);
          if (!in) a[u] = b[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          x[h][0] += a[u].x; x[h][1] += a[u].y; x[h][2] += a[u].z; x[h][3] += a[u].w;
          x[h][4] += b[u].x; x[h][5] += b[u].y; x[h][6] += b[u].z; x[h][7] += b[u].w;
        }
      }
    } else {
      Vec8<T> v;
      v.load(qkv + at);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[h][e] = v.get(e);
    }
  }

  if (kind != 2) {
    const TW* w = kind == 0 ? qw : kw;
    float wv[8], c[8], sn[8];
    if (w != nullptr) {
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[e] = to_f32(w[i * 8 + e]);
    }
    if (rope != nullptr) {
      const int j0 = (i % (TPT / 2)) * 8;
      const float* cs = rope + (size_t)(live ? t : tokens - 1) * D + j0;
      const float4 c0 = *reinterpret_cast<const float4*>(cs), c1 = *reinterpret_cast<const float4*>(cs + 4);
      const float4 s0 = *reinterpret_cast<const float4*>(cs + D / 2), s1 = *reinterpret_cast<const float4*>(cs + D / 2 + 4);
      c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
      sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
    }
    const bool low = i < TPT / 2;
    const int slot = (kind == 1 && live) ? slots[t] : 0;
#pragma unroll
    for (int h = 0; h < HPB; ++h) {
      if (h >= hn) break;  // the same for the whole block
      if (w != nullptr) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[h][e] * x[h][e];
#pragma unroll
        for (int o = 1; o < TPT; o <<= 1) ss += __shfl_xor(ss, o, WAVE);
        const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[h][e] = x[h][e] * rstd * wv[e];
      }
      if (rope != nullptr) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float partner = __shfl_xor(x[h][e], TPT / 2, WAVE);
          x[h][e] = low ? x[h][e] * c[e] - partner * sn[e] : x[h][e] * c[e] + partner * sn[e];
        }
      }
      if (live) {
        Vec8<T> v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v.set(e, x[h][e]);
        if (kind == 0) {
          v.store(q_out + (size_t)t * q_out_stride + (size_t)(h0 + h) * D + i * 8);
        } else {
          v.store(kc + (((size_t)(slot / page_size) * Hkv + (h0 + h)) * page_size + (slot % page_size)) * D + i * 8);
        }
      }
    }
    return;
  }

  // Value heads: through LDS, then thread (d, run) writes tokens 8 run .. 8 run + 7 of head element d.
  const int d = threadIdx.x / RUNS, run = threadIdx.x % RUNS;
  const int tr = t0 + run * 8;
  const int n_live = min(8, tokens - tr);
  int sl[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) sl[e] = slots[max(0, min(tr + e, tokens - 1))];
  bool run_ok = n_live == 8 && (page_size % 8 == 0) && (sl[0] % 8 == 0);
#pragma unroll
  for (int e = 1; e < 8; ++e) run_ok = run_ok && sl[e] == sl[0] + e;
#pragma unroll
  for (int h = 0; h < HPB; ++h) {
    if (h >= hn) break;  // the same for the whole block
    if (h > 0) __syncthreads();  // the previous head has been read out
    {
      Vec8<T> v;
#pragma unroll
      for (int e = 0; e < 8; ++e) v.set(e, x[h][e]);
      v.store(&vt[tl][i * 8]);
    }
    __syncthreads();
    if (tr >= tokens) continue;
    const int kvh = h0 + h;
    if (run_ok) {
      Vec8<T> v;
#pragma unroll
      for (int e = 0; e < 8; ++e) v.set(e, to_f32(vt[run * 8 + e][d]));
      v.store(vc + (((size_t)(sl[0] / page_size) * Hkv + kvh) * D + d) * page_size + (sl[0] % page_size));
    } else {
      for (int e = 0; e < n_live; ++e)
        vc[(((size_t)(sl[e] / page_size) * Hkv + kvh) * D + d) * page_size + (sl[e] % page_size)] = vt[run * 8 + e][d];
    }
  }
}

// Source: qkv [tokens, (Hq + 2 Hkv) D], or (parts != nullptr) float partial sums [splits, tokens, (Hq + 2 Hkv) D] of it.
// Queries go to q_out [tokens, q_out_stride >= Hq D] (which may be qkv itself: in place). rope is the
// table of ms_rope_table for these tokens with half = rot / 2 (nullptr when rot == 0), pairing an MS_ROPE_*
// number (MS_UNSUPPORTED for any other).
extern "C" int ms_qk_norm_rope_store(const void* qkv, const float* parts, int splits, long long split_stride, void* q_out,
                                     int q_out_stride, int is_bf16, const int* slots, const void* qw, const void* kw,
                                     int w_is_bf16, float eps, const float* rope, int rot, int pairing, void* kc, void* vc,
                                     int tokens, int Hq, int Hkv, int D, int page_size, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if ((qkv == nullptr) == (parts == nullptr) || (parts != nullptr && splits < 1) || q_out == nullptr || q_out_stride < Hq * D)
    return MS_BAD_ARG;
  if (D <= 0 || D > MAX_HEAD_DIM || rot < 0 || rot > D || (rot & 1) || Hq <= 0 || Hkv <= 0 || page_size <= 0) return MS_BAD_ARG;
  if ((qw == nullptr) != (kw == nullptr)) return MS_BAD_ARG;
  if ((rot > 0) != (rope != nullptr)) return MS_BAD_ARG;
  if (rot > 0 && pairing != MS_ROPE_HALVES && pairing != MS_ROPE_ADJACENT) return MS_UNSUPPORTED;
  const int heads = slots ? Hq + 2 * Hkv : Hq;
  if ((heads + 3) / 4 > 65535 || heads > 65535) return MS_BAD_ARG;
  // The tile kernel moves 8 elements at a time: every row it touches must start on such a boundary.
  // Which kernel runs depends on the head's shape alone, never on the number of tokens: a token's
  // result is the same bit for bit in whatever step it comes.
  const bool tiled = (D == 64 || D == 128) && (rot == 0 || (rot == D && pairing == MS_ROPE_HALVES)) && q_out_stride % 8 == 0 &&
                     (parts == nullptr || split_stride % 4 == 0);
  if (tiled) {
    const int tok_per_block = 256 / (D / 8);
    // Many tokens: four heads of a kind per block (more loads in flight per thread, the rotation's
    // cosines and sines read once for the four). Few tokens: a block per head, for more blocks.
    const int hpb = tokens > 256 ? 4 : 1;
    const dim3 grid((tokens + tok_per_block - 1) / tok_per_block, (Hq + hpb - 1) / hpb + (slots ? 2 * ((Hkv + hpb - 1) / hpb) : 0));
#define LAUNCH_TILE(T, TW, DD, HH)                                                                                       \
  qk_norm_rope_store_tile_kernel<T, TW, DD, HH><<<grid, 256, 0, st>>>((const T*)qkv, parts, splits, (size_t)split_stride, \
                                                                       (T*)q_out, q_out_stride, slots, (const TW*)qw,     \
                                                                       (const TW*)kw, eps, rope, (T*)kc, (T*)vc, tokens,  \
                                                                       Hq, Hkv, page_size)
#define LAUNCH_TILE_D(T, TW)                                                 \
  if (D == 128 && hpb == 4) LAUNCH_TILE(T, TW, 128, 4);                      \
  else if (D == 128) LAUNCH_TILE(T, TW, 128, 1);                             \
  else if (hpb == 4) LAUNCH_TILE(T, TW, 64, 4);                              \
  else LAUNCH_TILE(T, TW, 64, 1)
    if (is_bf16 && w_is_bf16) { LAUNCH_TILE_D(bf16, bf16); }
    else if (is_bf16) { LAUNCH_TILE_D(bf16, float); }
    else if (w_is_bf16) { LAUNCH_TILE_D(float, bf16); }
    else { LAUNCH_TILE_D(float, float); }
#undef LAUNCH_TILE_D
#undef LAUNCH_TILE
    return launch_status();
  }
#define LAUNCH(T, TW)                                                                                                   \
  qk_norm_rope_store_kernel<T, TW><<<dim3(tokens, (heads + 3) / 4), 256, 0, st>>>(                                      \
      (const T*)qkv, parts, splits, (size_t)split_stride, (T*)q_out, q_out_stride, slots, (const TW*)qw, (const TW*)kw, \
      eps, rope, rot, pairing, (T*)kc, (T*)vc, Hq, Hkv, D, page_size, heads)
  if (is_bf16 && w_is_bf16) LAUNCH(bf16, bf16);
  else if (is_bf16) LAUNCH(bf16, float);
  else if (w_is_bf16) LAUNCH(float, bf16);
  else LAUNCH(float, float);
#undef LAUNCH
  return launch_status();
}
