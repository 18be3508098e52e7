// Prefill attention for bfloat16: portions of prompts (several new tokens per sequence) over the
// paged cache, causal and bottom-right aligned (the query at position p sees keys <= p, or the last
// `window` of them), online softmax in float32, both products on v_mfma_f32_16x16x32_bf16.
//
// Work item = (tile of consecutive new tokens of one sequence, KV head). A block of 4 waves owns
// 128 query rows = tokens x the G query heads of the group (row = token * G + head), so K and V are
// read once for the whole group; each wave owns 32 rows (two 16-row MFMA blocks). Keys are walked
// in tiles of 64 tokens staged in LDS: K as [token][D], V as [D][token] (it already lies transposed
// within each page). Operand roles as in the decode kernel:
//   S^T[token, row] : A = K tile (i = token),  B = Q (j = row)      -> a lane holds 4 tokens of one row
//   O[row, d]       : A = P (i = row, k = token), B = V^T (j = d)   -> those same values are its P operand
// blockIdx.x = tile * Hkv + kvh: with 8 KV heads every KV head stays on one XCD and its tiles share
// that XCD's L2.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;  // 16 bytes in flight

#define PAGE 16
#define TK 64      // keys per tile

// 16-byte chunks of a tile of TK keys: K [TK tokens][D] and V^T [D][TK tokens], spread over 256 threads.
template <int D>
__device__ __forceinline__ void fetch_tile(u32x4 (&kreg)[TK * (D / 8) / 256], u32x4 (&vreg)[(TK / PAGE) * D * 2 / 256],
                                           const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                                           const int* __restrict__ table, int t0, int last_pos, int Hkv, int kvh, int tid) {
#pragma unroll
  for (int i = 0; i < TK * (D / 8) / 256; ++i) {
    const int c = tid + i * 256;
    const int tok = c / (D / 8), dc = c % (D / 8);
    const int t = min(t0 + tok, last_pos);
    const int page = max(table[t / PAGE], 0);  // a page behind the window was given back: masked later
    kreg[i] = *reinterpret_cast<const u32x4*>(kc + (((size_t)page * Hkv + kvh) * PAGE + t % PAGE) * D + dc * 8);
  }
#pragma unroll
  for (int i = 0; i < (TK / PAGE) * D * 2 / 256; ++i) {
    const int c = tid + i * 256;
    const int pi = c / (2 * D), rem = c % (2 * D), d = rem / 2, half = rem % 2;
    const int t = min(t0 + pi * PAGE, last_pos);
    const int page = max(table[t / PAGE], 0);
    vreg[i] = *reinterpret_cast<const u32x4*>(vc + (((size_t)page * Hkv + kvh) * D + d) * PAGE + half * 8);
  }
}

template <int D>
__device__ __forceinline__ void stash_tile(const u32x4 (&kreg)[TK * (D / 8) / 256],
                                           const u32x4 (&vreg)[(TK / PAGE) * D * 2 / 256], bf16* ks, bf16* vs, int tid) {
  constexpr int KS = D + 8, VS = TK + 8;
#pragma unroll
  for (int i = 0; i < TK * (D / 8) / 256; ++i) {
    const int c = tid + i * 256;
    *reinterpret_cast<u32x4*>(&ks[(c / (D / 8)) * KS + (c % (D / 8)) * 8]) = kreg[i];
  }
#pragma unroll
  for (int i = 0; i < (TK / PAGE) * D * 2 / 256; ++i) {
    const int c = tid + i * 256;
    const int pi = c / (2 * D), rem = c % (2 * D);
    *reinterpret_cast<u32x4*>(&vs[(rem / 2) * VS + pi * PAGE + (rem % 2) * 8]) = vreg[i];
  }
}

template <int D, int NQ>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ tile_first,
    const int* __restrict__ tile_count, const int* __restrict__ token_row, const int* __restrict__ pos,
    bf16* __restrict__ out, int Hq, int Hkv, float scale, int window) {
  constexpr int KK = D / 32, DB = D / 16;
  constexpr int ROWS = 64 * NQ;  // query rows per block: 16 NQ per wave
  constexpr int WROWS = 16 * NQ;
  constexpr int KS = D + 8;    // LDS row stride of the K tile (bf16)
  constexpr int VS = TK + 8;   // LDS row stride of the V^T tile
  __shared__ __attribute__((aligned(16))) bf16 ks[TK * KS];
  __shared__ __attribute__((aligned(16))) bf16 vs[D * VS];

  const int G = Hq / Hkv;
  const int kvh = blockIdx.x % Hkv, tile = blockIdx.x / Hkv;
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  const int first = tile_first[tile], count = tile_count[tile];
  const int pos0 = pos[first];
  const int* table = block_table + (size_t)token_row[first] * table_width;
  const int last_pos = pos0 + count - 1;
  const int kv_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;

  // This lane's query rows (one per 16-row block): token, position, validity.
  int row_tok[NQ], row_pos[NQ];
  bool row_ok[NQ];
  bf16x8 qf[NQ][KK];
#pragma unroll
  for (int b = 0; b < NQ; ++b) {
    const int row = wave * WROWS + b * 16 + r;
    row_tok[b] = row / G;
    row_ok[b] = row_tok[b] < count && row < (ROWS / G) * G;
    row_pos[b] = pos0 + row_tok[b];
    const int head = kvh * G + row % G;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (row_ok[b]) {
        qf[b][kk] = *reinterpret_cast<const bf16x8*>(q + (size_t)(first + row_tok[b]) * q_stride + (size_t)head * D + kk * 32 + g * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[b][kk][i] = static_cast<bf16>(0.f);
      }
    }
  }
  // Highest position among this wave's rows: tiles beyond it hold nothing the wave may see.
  const int wave_first_tok = (wave * WROWS) / G;
  const int wave_last_tok = min(count - 1, (wave * WROWS + WROWS - 1) / G);
  const bool wave_has_rows = wave_first_tok < count;
  const int wave_last_pos = pos0 + wave_last_tok;
  const int wave_first_pos = pos0 + wave_first_tok;

  float m_run[NQ], l_run[NQ];
  floatx4 o[NQ][DB];
#pragma unroll
  for (int b = 0; b < NQ; ++b) {
    m_run[b] = -INFINITY;
    l_run[b] = 0.f;
#pragma unroll
    for (int i = 0; i < DB; ++i) o[b][i] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // Global -> registers -> LDS, one tile ahead: the loads of tile i + 1 are in flight while tile i is
  // being multiplied. (A fetch past the last tile reads clamped, valid addresses and is dropped.)
  u32x4 kreg[TK * (D / 8) / 256], vreg[(TK / PAGE) * D * 2 / 256];
  const float scale2 = scale * 1.44269504088896340736f;  // scores in units of log2: exp2 is one instruction
  const int t_first = (kv_lo / TK) * TK;
  fetch_tile<D>(kreg, vreg, kc, vc, table, t_first, last_pos, Hkv, kvh, tid);
  for (int t0 = t_first; t0 <= last_pos; t0 += TK) {
    __syncthreads();  // the previous tile has been consumed
    stash_tile<D>(kreg, vreg, ks, vs, tid);
    __syncthreads();
    fetch_tile<D>(kreg, vreg, kc, vc, table, t0 + TK, last_pos, Hkv, kvh, tid);
    if (!wave_has_rows || t0 > wave_last_pos) continue;
    if (window > 0 && t0 + TK - 1 < wave_first_pos - window + 1) continue;

    floatx4 s[NQ][TK / 16];
#pragma unroll
    for (int b = 0; b < NQ; ++b)
#pragma unroll
      for (int tb = 0; tb < TK / 16; ++tb) s[b][tb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tb = 0; tb < TK / 16; ++tb) {
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(&ks[(tb * 16 + r) * KS + kk * 32 + g * 8]);
#pragma unroll
        for (int b = 0; b < NQ; ++b) s[b][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[b][kk], s[b][tb], 0, 0, 0);
      }
    }
    bf16x8 pf[NQ][TK / 32];
    float cq[NQ][4];
    // A tile needs masks only where it crosses the diagonal or the window's edge for some row of the wave.
    const bool masked = t0 + TK - 1 > wave_first_pos || (window > 0 && t0 <= wave_last_pos - window);
#pragma unroll
    for (int b = 0; b < NQ; ++b) {
      // Scores of row r of block b: tokens t0 + tb * 16 + 4 g + i.
      float m_new = m_run[b];
#pragma unroll
      for (int tb = 0; tb < TK / 16; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = s[b][tb][i] * scale2;
          if (masked) {
            const int t = t0 + tb * 16 + 4 * g + i;
            const bool seen = !row_ok[b] || (t <= row_pos[b] && (window == 0 || t > row_pos[b] - window));
            v = seen ? v : -INFINITY;
          }
          s[b][tb][i] = v;
          m_new = fmaxf(m_new, v);
        }
      m_new = fmaxf(m_new, __shfl_xor(m_new, 16, WAVE));
      m_new = fmaxf(m_new, __shfl_xor(m_new, 32, WAVE));
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
      float psum = 0.f;
#pragma unroll
      for (int tb = 0; tb < TK / 16; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __builtin_amdgcn_exp2f(s[b][tb][i] - m_safe);
          psum += p;
          pf[b][tb / 2][(tb % 2) * 4 + i] = static_cast<bf16>(p);
        }
      psum += __shfl_xor(psum, 16, WAVE);
      psum += __shfl_xor(psum, 32, WAVE);
      const float corr = __builtin_amdgcn_exp2f(m_run[b] - m_safe);
      l_run[b] = l_run[b] * corr + psum;
      m_run[b] = m_new;
#pragma unroll
      for (int i = 0; i < 4; ++i) cq[b][i] = __shfl(corr, 4 * g + i, WAVE);
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[b][db][i] *= cq[b][i];
    }
#pragma unroll
    for (int pr = 0; pr < TK / 32; ++pr) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16* vp = &vs[(db * 16 + r) * VS + pr * 32 + 4 * g];
        const bf16x4 va = *reinterpret_cast<const bf16x4*>(vp);
        const bf16x4 vb = *reinterpret_cast<const bf16x4*>(vp + 16);
        bf16x8 vf;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          vf[i] = va[i];
          vf[4 + i] = vb[i];
        }
#pragma unroll
        for (int b = 0; b < NQ; ++b) o[b][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[b][pr], vf, o[b][db], 0, 0, 0);
      }
    }
  }

  // o[b][db][i] = O[row 4 g + i of block b][d = db * 16 + r]
#pragma unroll
  for (int b = 0; b < NQ; ++b) {
    const float inv = 1.f / l_run[b];  // of row r; the rows written below are 4 g + i
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float inv_i = __shfl(inv, 4 * g + i, WAVE);
      const int row = wave * WROWS + b * 16 + 4 * g + i;
      const int tok = row / G;
      if (tok < count && row < (ROWS / G) * G) {
        bf16* dst = out + ((size_t)(first + tok) * Hq + kvh * G + row % G) * D;
#pragma unroll
        for (int db = 0; db < DB; ++db) dst[db * 16 + r] = static_cast<bf16>(o[b][db][i] * inv_i);
      }
    }
  }
}

// Query rows per block: 128 (two 16-row blocks per wave) when that still gives every CU two blocks,
// else 64. Tokens per tile = rows / G.
extern "C" int ms_attention_prefill_tile_tokens(int G, int rows) { return G >= 1 && G <= rows ? rows / G : 0; }

extern "C" int ms_attention_prefill_bf16(const void* q, int q_stride, const void* kc, const void* vc,
                                         const int* block_table, int table_width, const int* tile_first,
                                         const int* tile_count, int tiles, int rows_per_tile, const int* token_row,
                                         const int* pos, void* out, int Hq, int Hkv, int D, int page_size, float scale,
                                         int window, hipStream_t st) {
  if (tiles <= 0) return MS_OK;
  if (page_size != PAGE || (D != 64 && D != 128)) return MS_UNSUPPORTED;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hq / Hkv > 64 || window < 0 || table_width <= 0 || q_stride < Hq * D ||
      q_stride % 8 || (long long)tiles * Hkv > 2147483647LL || (rows_per_tile != 64 && rows_per_tile != 128))
    return MS_BAD_ARG;
  const unsigned grid = (unsigned)tiles * Hkv;
#define LAUNCH(DD, NN)                                                                                                  \
  attn_prefill_kernel<DD, NN><<<grid, 256, 0, st>>>((const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc,         \
                                                    block_table, table_width, tile_first, tile_count, token_row, pos,   \
                                                    (bf16*)out, Hq, Hkv, scale, window)
  if (D == 128 && rows_per_tile == 128) LAUNCH(128, 2);
  else if (D == 128) LAUNCH(128, 1);
  else if (rows_per_tile == 128) LAUNCH(64, 2);
  else LAUNCH(64, 1);
#undef LAUNCH
  return launch_status();
}
