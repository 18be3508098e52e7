// Prefill attention for bfloat16: portions of prompts (several new tokens per sequence) over the
// paged cache, causal and bottom-right aligned (the query at position p sees keys <= p, or the last
// `window` of them), online softmax in float32, both products on v_mfma_f32_16x16x32_bf16.
//
// Work item = (tile of consecutive new tokens of one sequence, KV head). A block owns 64 NQ query
// rows = tokens x the G query heads of the group (row = token * G + head), so K and V are read once
// for the whole group. Keys are walked in tiles of 64 tokens staged in LDS: K as [token][D], V as
// [D][token] (it already lies transposed within each page); page ids are fetched one tile ahead of
// the tile's loads, the loads one tile ahead of the products. Operand roles as in the decode kernel:
//   S^T[token, row] : A = K tile (i = token),  B = Q (j = row)      -> a lane holds 4 tokens of one row
//   O[row, d]       : A = P (i = row, k = token), B = V^T (j = d)   -> those same values are its P operand
// Waves: 4 row groups of 16 NQ rows, times KSPLIT key groups. With KSPLIT == 2 two waves share a row
// group and each takes half of every key tile (keeping its own running maximum, sum and output,
// merged once at the end): a prompt of a few thousand tokens has too few tiles to fill the chip, and
// its time is the longest tile's chain of iterations; halving the work per wave and iteration
// shortens that chain.
// blockIdx.x = tile * Hkv + kvh: with 8 KV heads every KV head stays on one XCD and its tiles share
// that XCD's L2.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;  // 16 bytes in flight
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4;

#define PAGE 16
#define TK 64  // keys per tile: four pages

// Page ids of the four pages of the key tile that starts at t0 (a multiple of TK): one 16-byte load
// (the table's width is a multiple of 4). Tiles past the last key are clamped to the last tile: what
// is fetched for them is dropped.
__device__ __forceinline__ i32x4 tile_pages(const int* __restrict__ table, int t0, int last_pos) {
  const int idx = min(t0, (last_pos / TK) * TK) / PAGE;
  return *reinterpret_cast<const i32x4*>(table + idx);
}

// 16-byte chunks of a tile of TK keys, K [TK tokens][D] and V^T [D][TK tokens], spread over NT threads.
// A page holds 2 D chunks of K and as many of V^T; chunk c = tid + NT i lies in page c / (2 D) of the
// tile for both. Pages wholly past the last key (or given back behind a window) are replaced by a
// valid page: their keys are masked.
template <int D, int NT>
__device__ __forceinline__ void fetch_tile(u32x4 (&kreg)[TK * (D / 8) / NT], u32x4 (&vreg)[TK * (D / 8) / NT],
                                           const bf16* __restrict__ kc, const bf16* __restrict__ vc, i32x4 pages, int t0,
                                           int last_pos, int Hkv, int kvh, int tid) {
  constexpr int PP = NT / (2 * D);  // pages one pass of the block's threads covers
  static_assert(PP >= 1 && (TK / PAGE) % PP == 0, "head size and block size");
  const int t_eff = min(t0, (last_pos / TK) * TK);
  const int sub = tid / (2 * D), within = tid % (2 * D);
#pragma unroll
  for (int i = 0; i < (TK / PAGE) / PP; ++i) {
    int page = pages[i * PP];
#pragma unroll
    for (int k = 1; k < PP; ++k)
      if (sub == k) page = pages[i * PP + k];
    if (t_eff + (i * PP + sub) * PAGE > last_pos) page = pages[0];
    page = max(page, 0);
    kreg[i] = *reinterpret_cast<const u32x4*>(kc + (((size_t)page * Hkv + kvh) * PAGE + within / (D / 8)) * D + (within % (D / 8)) * 8);
    vreg[i] = *reinterpret_cast<const u32x4*>(vc + (((size_t)page * Hkv + kvh) * D + within / 2) * PAGE + (within % 2) * 8);
  }
}

template <int D, int NT>
__device__ __forceinline__ void stash_tile(const u32x4 (&kreg)[TK * (D / 8) / NT], const u32x4 (&vreg)[TK * (D / 8) / NT],
                                           bf16* ks, bf16* vs, int tid) {
  constexpr int KS = D + 8, VS = TK + 8;
#pragma unroll
  for (int i = 0; i < TK * (D / 8) / NT; ++i) {
    const int c = tid + i * NT;
    *reinterpret_cast<u32x4*>(&ks[(c / (D / 8)) * KS + (c % (D / 8)) * 8]) = kreg[i];
    const int pi = c / (2 * D), rem = c % (2 * D);
    *reinterpret_cast<u32x4*>(&vs[(rem / 2) * VS + pi * PAGE + (rem % 2) * 8]) = vreg[i];
  }
}

template <int D, int NQ, int KSPLIT>
__global__ __launch_bounds__(256 * KSPLIT, 2 / KSPLIT) void attn_prefill_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ tile_first,
    const int* __restrict__ tile_count, const int* __restrict__ token_row, const int* __restrict__ pos,
    bf16* __restrict__ out, int Hq, int Hkv, float scale, int window) {
  constexpr int NT = 256 * KSPLIT;
  constexpr int KK = D / 32, DB = D / 16;
  constexpr int ROWS = 64 * NQ;     // query rows per block
  constexpr int WROWS = 16 * NQ;    // per row group
  constexpr int WK = TK / KSPLIT;   // keys of a tile per wave
  constexpr int TB = WK / 16;       // 16-key blocks per wave and tile
  constexpr int KS = D + 8;         // LDS row stride of the K tile (bf16)
  constexpr int VS = TK + 8;        // LDS row stride of the V^T tile
  // After the last tile the same memory carries the second key group's results to the first.
  constexpr int TILE_BYTES = (TK * KS + D * VS) * 2;
  constexpr int MERGE_BYTES = KSPLIT > 1 ? 4 * NQ * (16 * (D + 1) + 32) * 4 : 0;
  __shared__ __attribute__((aligned(16))) char smem[TILE_BYTES > MERGE_BYTES ? TILE_BYTES : MERGE_BYTES];
  bf16* ks = reinterpret_cast<bf16*>(smem);
  bf16* vs = ks + TK * KS;

  const int G = Hq / Hkv;
  const int kvh = blockIdx.x % Hkv, tile = blockIdx.x / Hkv;
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int rg = wave % 4, kg = wave / 4;  // row group, key group
  const int r = lane % 16, g = lane / 16;
  const int first = tile_first[tile], count = tile_count[tile];
  const int pos0 = pos[first];
  const int* table = block_table + (size_t)token_row[first] * table_width;
  const int last_pos = pos0 + count - 1;
  const int kv_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;

  // This lane's query rows (one per 16-row block): token, position, validity.
  int row_pos[NQ];
  bool row_ok[NQ];
  bf16x8 qf[NQ][KK];
#pragma unroll
  for (int b = 0; b < NQ; ++b) {
    const int row = rg * WROWS + b * 16 + r;
    const int tok = row / G;
    row_ok[b] = tok < count && row < (ROWS / G) * G;
    row_pos[b] = pos0 + tok;
    const int head = kvh * G + row % G;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (row_ok[b]) {
        qf[b][kk] = *reinterpret_cast<const bf16x8*>(q + (size_t)(first + tok) * q_stride + (size_t)head * D + kk * 32 + g * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[b][kk][i] = static_cast<bf16>(0.f);
      }
    }
  }
  // Lowest and highest position among this row group's rows: tiles beyond them hold nothing it may see.
  const int grp_first_tok = (rg * WROWS) / G;
  const int grp_last_tok = min(count - 1, (rg * WROWS + WROWS - 1) / G);
  const bool grp_has_rows = grp_first_tok < count;
  const int grp_last_pos = pos0 + grp_last_tok;
  const int grp_first_pos = pos0 + grp_first_tok;

  float m_run[NQ], l_run[NQ];
  floatx4 o[NQ][DB];
#pragma unroll
  for (int b = 0; b < NQ; ++b) {
    m_run[b] = -INFINITY;
    l_run[b] = 0.f;
#pragma unroll
    for (int i = 0; i < DB; ++i) o[b][i] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // Global -> registers -> LDS with PD tiles in flight: a tile's loads are issued PD iterations before
  // it is needed, since one iteration of products is much shorter than a trip to memory. The register
  // sets rotate; the loop is unrolled PD-fold so that each set has a fixed name.
  constexpr int PD = (KSPLIT == 1 && D == 128) ? 1 : 3;  // the widest variant has no registers to spare
  u32x4 kreg[PD][TK * (D / 8) / NT], vreg[PD][TK * (D / 8) / NT];
  const float scale2 = scale * 1.44269504088896340736f;  // scores in units of log2: exp2 is one instruction
  const int t_first = (kv_lo / TK) * TK;
#pragma unroll
  for (int st = 0; st < PD; ++st)
    fetch_tile<D, NT>(kreg[st], vreg[st], kc, vc, tile_pages(table, t_first + st * TK, last_pos), t_first + st * TK, last_pos,
                      Hkv, kvh, tid);
  i32x4 pages_next = tile_pages(table, t_first + PD * TK, last_pos);
  for (int tbase = t_first; tbase <= last_pos; tbase += PD * TK) {
#pragma unroll
  for (int st = 0; st < PD; ++st) {
    const int t0 = tbase + st * TK;
    if (t0 > last_pos) break;
    __syncthreads();  // the previous tile has been consumed
    stash_tile<D, NT>(kreg[st], vreg[st], ks, vs, tid);
    __syncthreads();
    fetch_tile<D, NT>(kreg[st], vreg[st], kc, vc, pages_next, t0 + PD * TK, last_pos, Hkv, kvh, tid);
    pages_next = tile_pages(table, t0 + (PD + 1) * TK, last_pos);
    const int w0 = t0 + kg * WK;  // this wave's keys of the tile: w0 .. w0 + WK - 1
    if (!grp_has_rows || w0 > grp_last_pos) continue;
    if (window > 0 && w0 + WK - 1 < grp_first_pos - window + 1) continue;

    floatx4 s[NQ][TB];
#pragma unroll
    for (int b = 0; b < NQ; ++b)
#pragma unroll
      for (int tb = 0; tb < TB; ++tb) s[b][tb] = floatx4{0.f, 0.f, 0.f, 0.f};
    {
      // All K fragments are requested from LDS before the first product is issued: the reads return
      // in order, so each product waits only for its own operand while the rest are in flight.
      bf16x8 kf[TB][KK];
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
          kf[tb][kk] = *reinterpret_cast<const bf16x8*>(&ks[(kg * WK + tb * 16 + r) * KS + kk * 32 + g * 8]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)  // consecutive products go to different accumulators
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
          for (int b = 0; b < NQ; ++b) s[b][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[tb][kk], qf[b][kk], s[b][tb], 0, 0, 0);
    }
    bf16x8 pf[NQ][TB / 2];
    // Masks only where the keys cross the diagonal or the window's edge for some row of the group.
    const bool masked = w0 + WK - 1 > grp_first_pos || (window > 0 && w0 <= grp_last_pos - window);
#pragma unroll
    for (int b = 0; b < NQ; ++b) {
      // Scores of row r of block b: tokens w0 + tb * 16 + 4 g + i.
      float m_new = m_run[b];
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = s[b][tb][i] * scale2;
          if (masked) {
            const int t = w0 + tb * 16 + 4 * g + i;
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
      for (int tb = 0; tb < TB; ++tb)
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
      float cq[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) cq[i] = __shfl(corr, 4 * g + i, WAVE);
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[b][db][i] *= cq[i];
    }
    {
      // The same for the V^T fragments of the second product.
      bf16x4 va[TB / 2][DB], vb[TB / 2][DB];
#pragma unroll
      for (int pr = 0; pr < TB / 2; ++pr)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const bf16* vp = &vs[(db * 16 + r) * VS + kg * WK + pr * 32 + 4 * g];
          va[pr][db] = *reinterpret_cast<const bf16x4*>(vp);
          vb[pr][db] = *reinterpret_cast<const bf16x4*>(vp + 16);
        }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int pr = 0; pr < TB / 2; ++pr)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          bf16x8 vf;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            vf[i] = va[pr][db][i];
            vf[4 + i] = vb[pr][db][i];
          }
#pragma unroll
          for (int b = 0; b < NQ; ++b) o[b][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[b][pr], vf, o[b][db], 0, 0, 0);
        }
    }
  }
  }

  if (KSPLIT > 1) {
    // The second key group hands its running maximum, sum and output to the first through LDS.
    // Layout per (row group, block): 16 rows x (D + 1) floats of output, then 16 maxima, then 16 sums.
    __syncthreads();  // the last tile has been consumed
    float* mg = reinterpret_cast<float*>(smem);
    constexpr int PER = 16 * (D + 1) + 32;
#pragma unroll
    for (int b = 0; b < NQ; ++b) {
      float* base = mg + (rg * NQ + b) * PER;
      if (kg == 1) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) base[(4 * g + i) * (D + 1) + db * 16 + r] = o[b][db][i];
        if (g == 0) {
          base[16 * (D + 1) + r] = m_run[b];
          base[16 * (D + 1) + 16 + r] = l_run[b];
        }
      }
    }
    __syncthreads();
    if (kg == 1) return;
#pragma unroll
    for (int b = 0; b < NQ; ++b) {
      const float* base = mg + (rg * NQ + b) * PER;
      const float m2 = base[16 * (D + 1) + r], l2 = base[16 * (D + 1) + 16 + r];
      const float m = fmaxf(m_run[b], m2);
      const float m_safe = m == -INFINITY ? 0.f : m;
      const float f1 = __builtin_amdgcn_exp2f(m_run[b] - m_safe), f2 = __builtin_amdgcn_exp2f(m2 - m_safe);
      l_run[b] = l_run[b] * f1 + l2 * f2;
      m_run[b] = m;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a1 = __shfl(f1, 4 * g + i, WAVE), a2 = __shfl(f2, 4 * g + i, WAVE);
#pragma unroll
        for (int db = 0; db < DB; ++db) o[b][db][i] = o[b][db][i] * a1 + base[(4 * g + i) * (D + 1) + db * 16 + r] * a2;
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
      const int row = rg * WROWS + b * 16 + 4 * g + i;
      const int tok = row / G;
      if (tok < count && row < (ROWS / G) * G) {
        bf16* dst = out + ((size_t)(first + tok) * Hq + kvh * G + row % G) * D;
#pragma unroll
        for (int db = 0; db < DB; ++db) dst[db * 16 + r] = static_cast<bf16>(o[b][db][i] * inv_i);
      }
    }
  }
}

// Tokens per tile for a group of G query heads per KV head and `rows` query rows per block.
extern "C" int ms_attention_prefill_tile_tokens(int G, int rows) { return G >= 1 && G <= rows ? rows / G : 0; }

// rows_per_tile: 128 (large batches of tiles: least traffic per product) or 64 (each wave then takes
// half of every key tile: shortest chain per tile).
extern "C" int ms_attention_prefill_bf16(const void* q, int q_stride, const void* kc, const void* vc,
                                         const int* block_table, int table_width, const int* tile_first,
                                         const int* tile_count, int tiles, int rows_per_tile, const int* token_row,
                                         const int* pos, void* out, int Hq, int Hkv, int D, int page_size, float scale,
                                         int window, hipStream_t st) {
  if (tiles <= 0) return MS_OK;
  if (page_size != PAGE || (D != 64 && D != 128)) return MS_UNSUPPORTED;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hq / Hkv > 64 || window < 0 || table_width <= 0 || table_width % 4 ||
      q_stride < Hq * D || q_stride % 8 || (long long)tiles * Hkv > 2147483647LL ||
      (rows_per_tile != 64 && rows_per_tile != 128))
    return MS_BAD_ARG;
  const unsigned grid = (unsigned)tiles * Hkv;
#define LAUNCH(DD, NN, KS_)                                                                                       \
  attn_prefill_kernel<DD, NN, KS_><<<grid, 256 * KS_, 0, st>>>((const bf16*)q, q_stride, (const bf16*)kc,         \
                                                               (const bf16*)vc, block_table, table_width,         \
                                                               tile_first, tile_count, token_row, pos,            \
                                                               (bf16*)out, Hq, Hkv, scale, window)
  if (D == 128 && rows_per_tile == 128) LAUNCH(128, 2, 1);
  else if (D == 128) LAUNCH(128, 1, 2);
  else if (rows_per_tile == 128) LAUNCH(64, 2, 1);
  else LAUNCH(64, 1, 2);
#undef LAUNCH
  return launch_status();
}
