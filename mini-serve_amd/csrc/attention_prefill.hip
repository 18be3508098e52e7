// Prefill attention for bfloat16: portions of prompts (several new tokens per sequence) over the
// paged cache, causal and bottom-right aligned (the query at position p sees keys <= p, or the last
// `window` of them), online softmax in float32, both products on v_mfma_f32_16x16x32_bf16.
//
// Work item = (tile of consecutive new tokens of one sequence, KV head). A block owns 64 NQ query
// rows = tokens x the G query heads of the group (row = token * G + head), so K and V are read once
// for the whole group. Keys are walked in tiles of 64 tokens held in LDS: K as [token][D], V as
// [D][token] (it already lies transposed within each page). The tiles go straight from the cache pages
// into a ring of LDS stages (global_load_lds, 16 bytes per lane, no staging registers and no LDS
// stores), each row's 16-byte chunks permuted so that the fragment reads touch every bank once; page
// ids are fetched one tile ahead of the tile's loads, the loads STAGES - 1 tiles ahead of the
// products, and there is one barrier per tile. Operand roles as in the decode kernel:
//   S^T[token, row] : A = K tile (i = token),  B = Q (j = row)
//   O^T[d, row]     : A = V^T (i = d, k = token), B = P (j = row)   -> a lane's outputs are of its own row,
//                                                                      whose maximum and sum it holds
// The key rows of the two score products of a 32-key pair are taken in an order that leaves a lane
// with 8 consecutive keys of one page: exactly its P operand, and its V^T operand is one 16-byte read.
// Waves: 4 row groups of 16 NQ rows, times KSPLIT key groups. With KSPLIT == 2 two waves share a row
// group and each takes half of every key tile (keeping its own running maximum, sum and output,
// merged once at the end): a prompt of a few thousand tokens has too few tiles to fill the chip, and
// its time is the longest tile's chain of iterations; halving the work per wave and iteration
// shortens that chain.
// blockIdx.x = tile * Hkv + kvh: with 8 KV heads every KV head stays on one XCD and its tiles share
// that XCD's L2.
//
// A batch with few tiles (one short prompt) leaves the chip to the deepest tile's chain of iterations,
// which runs on alone when every other block is done. The host may therefore hand a tile's keys out in
// parts: an entry then names a range of key tiles and a slot, the block leaves its running maximum,
// sum and unnormalised output there, and a second kernel merges a tile's parts in ascending order.
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

// Wait until at most N of this wave's vector-memory loads are in flight (expcnt and lgkmcnt are left alone).
template <int N>
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// v[i] by three selects (no branch): i differs between the lanes of a wave.
__device__ __forceinline__ int pick(i32x4 v, int i) {
  int p = v[0];
  p = i == 1 ? v[1] : p;
  p = i == 2 ? v[2] : p;
  p = i == 3 ? v[3] : p;
  return p;
}

template <int D, int NQ, int KSPLIT, int STAGES, int BLOCKS_PER_CU>
// (the second launch bound counts waves per SIMD: a block of 256 KSPLIT threads puts KSPLIT on each)
__global__ __launch_bounds__(256 * KSPLIT, BLOCKS_PER_CU * KSPLIT) void attn_prefill_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ tile_first,
    const int* __restrict__ tile_count, const int* __restrict__ token_row, const int* __restrict__ pos,
    bf16* __restrict__ out, int Hq, int Hkv, float scale, int window, const int* __restrict__ tile_key_begin,
    const int* __restrict__ tile_key_end, const int* __restrict__ tile_slot, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  constexpr int NT = 256 * KSPLIT, NW = NT / WAVE;
  constexpr int KK = D / 32, DB = D / 16;
  constexpr int ROWS = 64 * NQ;     // query rows per block
  constexpr int WROWS = 16 * NQ;    // per row group
  constexpr int WK = TK / KSPLIT;   // keys of a tile per wave
  constexpr int TB = WK / 16;       // 16-key blocks per wave and tile
  constexpr int KROW = D * 2;       // bytes of a K row in LDS (no padding: the chunks are permuted instead)
  constexpr int KCH = D / 8;        // its 16-byte chunks: 8 or 16
  constexpr int KRPI = 1024 / KROW; // K rows one load instruction of a wave fills
  constexpr int KI = TK / KRPI / NW;  // K load instructions per wave and tile
  constexpr int VROW = TK * 2;      // bytes of a V^T row (one head element, 64 keys)
  constexpr int VI = D / 8 / NW;    // V^T load instructions per wave and tile (8 rows each)
  constexpr int K_BYTES = TK * KROW, STAGE_BYTES = K_BYTES + D * VROW;
  static_assert(KI >= 1 && VI >= 1 && KI * KRPI * NW == TK && VI * 8 * NW == D, "head size and block size");
  // After the last tile the same memory carries the second key group's results to the first.
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];  // prefill_lds_bytes<D, NQ, KSPLIT, STAGES>()

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

  // Chunk c of K row R lies in slot c ^ kswz(R) of the row, chunk c of V^T row d in slot c ^ ((d >> 1) & 7).
  // The 16 lanes that read a chunk column together take key rows {0-3, 8-11, 16-19, 24-27} (+ 4, + 32):
  // the rows differ in bits 0, 1, 3 and 4, and it is these that must give 16 different slots (a
  // 256-byte row starts at bank 0; with 128-byte rows bit 0 already picks the half of the banks).
  auto kswz = [](int R) { return KCH == 16 ? ((R & 3) | ((R >> 1) & 12)) : (((R >> 1) & 1) | ((R >> 2) & 6)); };
  // One tile's loads: wave-instruction q fills 1 KB of the stage in lane order. What does not depend on
  // the tile is worked out once: the offset of the lane's chunk within its page, and which of the
  // tile's four pages it comes from. Tiles past the last key are clamped to the last tile (what is
  // fetched for them is never used); table entries without a page (past the last key, or given back
  // behind a window) read page 0 instead: their keys are masked.
  const size_t page_elems = (size_t)Hkv * PAGE * D;  // one page of K, and of V^T
  int k_page[KI], v_page[VI];
  unsigned k_off[KI], v_off[VI];
#pragma unroll
  for (int j = 0; j < KI; ++j) {
    const int R = (wave * KI + j) * KRPI + lane / KCH, c = (lane % KCH) ^ kswz(R);
    k_page[j] = __builtin_amdgcn_readfirstlane(R / PAGE);  // the rows of one instruction lie in one page
    k_off[j] = (unsigned)((kvh * PAGE + R % PAGE) * D + c * 8);
  }
#pragma unroll
  for (int j = 0; j < VI; ++j) {
    const int d = (wave * VI + j) * 8 + lane / 8, c = (lane % 8) ^ ((d >> 1) & 7);  // chunk c: keys 8 c .. 8 c + 7 of the tile
    v_page[j] = c / 2;
    v_off[j] = (unsigned)((kvh * D + d) * PAGE + (c % 2) * 8);
  }
  auto issue = [&](i32x4 pages, int stage_index) __attribute__((always_inline)) {
    unsigned char* stage = smem + stage_index * STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < KI; ++j) {
      const bf16* src = kc + (size_t)max(pick(pages, k_page[j]), 0) * page_elems + k_off[j];
      __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)src,
                                       (void __attribute__((address_space(3)))*)(stage + (wave * KI + j) * 1024), 16, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < VI; ++j) {
      const bf16* src = vc + (size_t)max(pick(pages, v_page[j]), 0) * page_elems + v_off[j];
      __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)src,
                                       (void __attribute__((address_space(3)))*)(stage + K_BYTES + (wave * VI + j) * 1024), 16,
                                       0, 0);
    }
  };

  const float scale2 = scale * 1.44269504088896340736f;  // scores in units of log2: exp2 is one instruction
  // The key tiles this block visits: all the tile's rows may see, or the part the host names (in units
  // of key tiles from position 0; the host leaves no part empty).
  const int slot = tile_slot ? tile_slot[tile] : -1;
  const int t_first = max((kv_lo / TK) * TK, tile_key_begin ? tile_key_begin[tile] * TK : 0);
  const int key_last = tile_key_end ? min(last_pos, tile_key_end[tile] * TK - 1) : last_pos;
  const int n_tiles = (key_last - t_first) / TK + 1;
  // Issue order: page ids of tile m + 1, then the loads of tile m. At the top of iteration n the loads
  // of tiles n + 1 .. n + STAGES - 2 may still be in flight, those of tile n must have landed.
  i32x4 pages_next = tile_pages(table, t_first, last_pos);
#pragma unroll
  for (int st = 0; st < STAGES - 1; ++st) {
    const i32x4 pages = pages_next;
    pages_next = tile_pages(table, t_first + (st + 1) * TK, last_pos);
    issue(pages, st);
  }
  // This lane's key rows of a 32-key pair: product h (0 or 1) takes keys 4 h + {0-3, 8-11} of each of
  // the pair's two pages, rows 0-7 from the first page and 8-15 from the second.
  const int krow = (r < 8 ? 0 : 16) + (r % 4) + 8 * ((r / 4) % 2);
  const int vsw = (r >> 1) & 7;
  for (int n = 0; n < n_tiles; ++n) {
    const int t0 = t_first + n * TK;
    wait_loads<(STAGES - 2) * (KI + VI)>();
    __syncthreads();  // tile n has landed for every wave, and every wave is done with tile n - 1
    {
      const i32x4 pages = pages_next;
      pages_next = tile_pages(table, t0 + STAGES * TK, last_pos);
      issue(pages, (n + STAGES - 1) % STAGES);
    }
    const unsigned char* ks = smem + (n % STAGES) * STAGE_BYTES;
    const unsigned char* vs = ks + K_BYTES;
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
        {
          const int R = kg * WK + (tb / 2) * 32 + krow + 4 * (tb % 2);
          kf[tb][kk] = *reinterpret_cast<const bf16x8*>(ks + R * KROW + (((kk * 4 + g) ^ kswz(R)) * 16));
        }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)  // consecutive products go to different accumulators
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
          for (int b = 0; b < NQ; ++b) s[b][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[tb][kk], qf[b][kk], s[b][tb], 0, 0, 0);
    }
    bf16x8 pf[NQ][TB / 2];
    // Masks only where the keys cross the diagonal or the window's edge for some row of the group
    // (the same answer for the whole wave: one branch around all of it).
    const bool masked = __builtin_amdgcn_readfirstlane(
        (int)(w0 + WK - 1 > grp_first_pos || (window > 0 && w0 <= grp_last_pos - window)));
    if (masked) {
#pragma unroll
      for (int b = 0; b < NQ; ++b)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            // Scores of row r of block b: keys w0 + (tb / 2) * 32 + 8 g + 4 (tb % 2) + i.
            const int t = w0 + (tb / 2) * 32 + 8 * g + 4 * (tb % 2) + i;
            const bool seen = !row_ok[b] | ((t <= row_pos[b]) & ((window == 0) | (t > row_pos[b] - window)));
            s[b][tb][i] = seen ? s[b][tb][i] : -INFINITY;
          }
    }
#pragma unroll
    for (int b = 0; b < NQ; ++b) {
      // The maximum is taken over the raw scores (the scale is positive) and scaled once; the scale
      // itself enters in the exponent's fused multiply-add. -inf stays -inf through both.
      float s_max = -INFINITY;
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_max = fmaxf(s_max, s[b][tb][i]);
      const float m_new = fmaxf(m_run[b], rows4_max(s_max) * scale2);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
      float psum = 0.f;
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[b][tb][i], scale2, -m_safe));
          psum += p;
          pf[b][tb / 2][(tb % 2) * 4 + i] = static_cast<bf16>(p);
        }
      psum = rows4_sum(psum);
      const float corr = __builtin_amdgcn_exp2f(m_run[b] - m_safe);
      l_run[b] = l_run[b] * corr + psum;
      m_run[b] = m_new;
      // Once the maxima of a wave's rows have settled (after the first few tiles, as a rule) the
      // correction is exactly 1 for all of them, and the output is left alone.
      if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[b][db][i] *= corr;  // the lane's output values are all of its own row
      }
    }
    {
      // The same for the V^T fragments of the second product: keys 8 g .. 8 g + 7 of the pair.
      bf16x8 vf[TB / 2][DB];
#pragma unroll
      for (int pr = 0; pr < TB / 2; ++pr)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int c = (kg * WK + pr * 32) / 8 + g;
          vf[pr][db] = *reinterpret_cast<const bf16x8*>(vs + (db * 16 + r) * VROW + ((c ^ vsw) * 16));
        }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int pr = 0; pr < TB / 2; ++pr)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int b = 0; b < NQ; ++b) o[b][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[pr][db], pf[b][pr], o[b][db], 0, 0, 0);
    }
  }
  wait_loads<0>();  // the tiles fetched ahead past the end must not land in memory that is used otherwise

  if (KSPLIT > 1) {
    // The second key group hands its running maximum, sum and output to the first through LDS.
    // Layout per (row group, block): 16 rows x (D + 1) floats of output, then 16 maxima, then 16 sums.
    __syncthreads();  // the last tile has been consumed, and nothing is in flight any more
    float* mg = reinterpret_cast<float*>(smem);
    constexpr int PER = 16 * (D + 1) + 32;
#pragma unroll
    for (int b = 0; b < NQ; ++b) {
      float* base = mg + (rg * NQ + b) * PER;
      if (kg == 1) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) base[r * (D + 1) + db * 16 + 4 * g + i] = o[b][db][i];
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
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[b][db][i] = o[b][db][i] * f1 + base[r * (D + 1) + db * 16 + 4 * g + i] * f2;
    }
  }

  // o[b][db][i] = O[row r of block b][d = db * 16 + 4 g + i]
  if (slot >= 0) {
    // A part of the tile's keys: maximum, sum and unnormalised output of every row go to the slot.
    const size_t base = ((size_t)slot * Hkv + kvh) * ROWS;
#pragma unroll
    for (int b = 0; b < NQ; ++b) {
      const int row = rg * WROWS + b * 16 + r;
      float* po = part_o + (base + row) * D + 4 * g;
#pragma unroll
      for (int db = 0; db < DB; ++db) *reinterpret_cast<floatx4*>(po + db * 16) = o[b][db];
      if (g == 0) {
        part_ml[(base + row) * 2] = m_run[b];
        part_ml[(base + row) * 2 + 1] = l_run[b];
      }
    }
    return;
  }
#pragma unroll
  for (int b = 0; b < NQ; ++b) {
    const float inv = 1.f / l_run[b];
    const int row = rg * WROWS + b * 16 + r;
    const int tok = row / G;
    if (tok < count && row < (ROWS / G) * G) {
      bf16* dst = out + ((size_t)(first + tok) * Hq + kvh * G + row % G) * D + 4 * g;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = static_cast<bf16>(o[b][db][i] * inv);
        *reinterpret_cast<bf16x4*>(dst + db * 16) = v;
      }
    }
  }
}

// Merges the parts of the tiles whose keys were handed out in parts: grid (merged tiles, Hkv, groups of
// 16 rows). A tile's
// parts lie in consecutive slots, in ascending order of their keys, and are added in that order. A part
// in which a row saw no key (behind its window) has maximum -inf and adds nothing.
template <int D>
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(const int* __restrict__ merge_first,
                                                                 const int* __restrict__ merge_count,
                                                                 const int* __restrict__ merge_slot,
                                                                 const int* __restrict__ merge_parts,
                                                                 const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml, bf16* __restrict__ out,
                                                                 int Hq, int Hkv, int rows) {
  const int t = blockIdx.x, kvh = blockIdx.y;
  const int G = Hq / Hkv;
  const int first = merge_first[t], count = merge_count[t], slot0 = merge_slot[t], parts = merge_parts[t];
  const int used = min(count * G, (rows / G) * G);  // rows of the tile that hold a token's head
  const int row_end = min(used, (int)(blockIdx.z + 1) * 16);
  for (int idx = blockIdx.z * 16 * (D / 4) + threadIdx.x; idx < row_end * (D / 4); idx += 256) {
    const int row = idx / (D / 4), d = (idx % (D / 4)) * 4;
    float m = -INFINITY;
    for (int p = 0; p < parts; ++p) m = fmaxf(m, part_ml[(((size_t)(slot0 + p) * Hkv + kvh) * rows + row) * 2]);
    float l = 0.f;
    floatx4 o = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int p = 0; p < parts; ++p) {
      const size_t at = ((size_t)(slot0 + p) * Hkv + kvh) * rows + row;
      const float mp = part_ml[at * 2];
      const float f = mp == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mp - m);
      l += part_ml[at * 2 + 1] * f;
      const floatx4 v = *reinterpret_cast<const floatx4*>(part_o + at * D + d);
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] += v[i] * f;
    }
    const float inv = 1.f / l;
    bf16x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<bf16>(o[i] * inv);
    *reinterpret_cast<bf16x4*>(out + ((size_t)(first + row / G) * Hq + kvh * G + row % G) * D + d) = v;
  }
}

// What the host adds when it hands tiles' keys out in parts (all null / 0 otherwise).
struct PrefillParts {
  const int* key_begin;    // per entry: first key tile
  const int* key_end;      // per entry: one past its last key tile
  const int* slot;         // per entry: where its partial result goes, or -1: it is the whole tile
  float* part_o;           // [slots, Hkv, rows per tile, D]
  float* part_ml;          // [slots, Hkv, rows per tile, 2]
  const int* merge_first;  // per merged tile: first token, token count, first slot, number of parts
  const int* merge_count;
  const int* merge_slot;
  const int* merge_parts;
  int merges;
};

template <int D, int NQ, int KSPLIT, int STAGES>
constexpr int prefill_lds_bytes() {
  constexpr int tiles = STAGES * (TK * D * 2 + D * TK * 2);
  constexpr int merge = KSPLIT > 1 ? 4 * NQ * (16 * (D + 1) + 32) * 4 : 0;
  return tiles > merge ? tiles : merge;
}

template <int D, int NQ, int KSPLIT, int STAGES, int BLOCKS_PER_CU>
static int launch_prefill(unsigned grid, const bf16* q, int q_stride, const bf16* kc, const bf16* vc, const int* block_table,
                          int table_width, const int* tile_first, const int* tile_count, const int* token_row,
                          const int* pos, bf16* out, int Hq, int Hkv, float scale, int window, PrefillParts pp,
                          hipStream_t st) {
  constexpr int lds = prefill_lds_bytes<D, NQ, KSPLIT, STAGES>();
  static_assert(lds * BLOCKS_PER_CU <= 160 * 1024, "LDS of the blocks that share a CU");
  static bool ready = false;  // more than 64 KB of LDS has to be asked for once per kernel
  if (!ready) {
    if (hipFuncSetAttribute((const void*)attn_prefill_kernel<D, NQ, KSPLIT, STAGES, BLOCKS_PER_CU>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return MS_LAUNCH_FAILED;
    ready = true;
  }
  attn_prefill_kernel<D, NQ, KSPLIT, STAGES, BLOCKS_PER_CU><<<grid, 256 * KSPLIT, lds, st>>>(q, q_stride, kc, vc, block_table, table_width,
                                                                              tile_first, tile_count, token_row, pos, out,
                                                                              Hq, Hkv, scale, window, pp.key_begin, pp.key_end,
                                                                              pp.slot, pp.part_o, pp.part_ml);
  if (pp.merges > 0)
    attn_prefill_merge_kernel<D><<<dim3(pp.merges, Hkv, 4 * NQ), 256, 0, st>>>(pp.merge_first, pp.merge_count, pp.merge_slot,
                                                                       pp.merge_parts, pp.part_o, pp.part_ml, out, Hq, Hkv,
                                                                       64 * NQ);
  return launch_status();
}
#define PREFILL_ARGS                                                                                                    \
  (const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc, block_table, table_width, tile_first, tile_count, token_row, \
      pos, (bf16*)out, Hq, Hkv, scale, window, pp, st

// Tokens per tile for a group of G query heads per KV head and `rows` query rows per block.
extern "C" int ms_attention_prefill_tile_tokens(int G, int rows) { return G >= 1 && G <= rows ? rows / G : 0; }

// rows_per_tile: 128 (large batches of tiles: least traffic per product) or 64 (each wave then takes
// half of every key tile: shortest chain per tile).
static int prefill_dispatch(const void* q, int q_stride, const void* kc, const void* vc, const int* block_table,
                            int table_width, const int* tile_first, const int* tile_count, int tiles, int rows_per_tile,
                            const int* token_row, const int* pos, void* out, int Hq, int Hkv, int D, int page_size,
                            float scale, int window, PrefillParts pp, hipStream_t st) {
  if (tiles <= 0) return MS_OK;
  if (page_size != PAGE || (D != 64 && D != 128)) return MS_UNSUPPORTED;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hq / Hkv > 64 || window < 0 || table_width <= 0 || table_width % 4 ||
      q_stride < Hq * D || q_stride % 8 || (long long)tiles * Hkv > 2147483647LL ||
      (rows_per_tile != 64 && rows_per_tile != 128) || Hkv > 65535)
    return MS_BAD_ARG;
  const unsigned grid = (unsigned)tiles * Hkv;
  // Two stages were as fast as four in every shape tried (the loop is bound by its instructions, not
  // by the loads), and leave room for two blocks per CU.
  if (D == 128 && rows_per_tile == 128) return launch_prefill<128, 2, 1, 2, 2>(grid, PREFILL_ARGS);
  if (D == 128) return launch_prefill<128, 1, 2, 2, 2>(grid, PREFILL_ARGS);
  if (rows_per_tile == 128) return launch_prefill<64, 2, 1, 2, 2>(grid, PREFILL_ARGS);
  return launch_prefill<64, 1, 2, 2, 2>(grid, PREFILL_ARGS);
}

extern "C" int ms_attention_prefill_bf16(const void* q, int q_stride, const void* kc, const void* vc,
                                         const int* block_table, int table_width, const int* tile_first,
                                         const int* tile_count, int tiles, int rows_per_tile, const int* token_row,
                                         const int* pos, void* out, int Hq, int Hkv, int D, int page_size, float scale,
                                         int window, hipStream_t st) {
  return prefill_dispatch(q, q_stride, kc, vc, block_table, table_width, tile_first, tile_count, tiles, rows_per_tile,
                          token_row, pos, out, Hq, Hkv, D, page_size, scale, window, PrefillParts{}, st);
}

// The same with tiles' keys handed out in parts. `plan` holds, as consecutive int arrays on the device:
// per entry (entries of them) first token, token count, first key tile, end key tile, slot (-1: the
// entry is a whole tile); then per merged tile (merges of them) first token, token count, first slot,
// number of parts. part_o holds slots * Hkv * rows_per_tile * D floats, part_ml slots * Hkv *
// rows_per_tile * 2. Only for layers without a window: the parts count key tiles from position 0.
extern "C" int ms_attention_prefill_parts_bf16(const void* q, int q_stride, const void* kc, const void* vc,
                                               const int* block_table, int table_width, const int* plan, int entries,
                                               int merges, float* part_o, float* part_ml, int rows_per_tile,
                                               const int* token_row, const int* pos, void* out, int Hq, int Hkv, int D,
                                               int page_size, float scale, hipStream_t st) {
  if (entries <= 0) return MS_OK;
  if (plan == nullptr || merges < 0 || (merges > 0 && (!part_o || !part_ml))) return MS_BAD_ARG;
  PrefillParts pp;
  pp.key_begin = plan + 2 * (size_t)entries;
  pp.key_end = plan + 3 * (size_t)entries;
  pp.slot = plan + 4 * (size_t)entries;
  pp.part_o = part_o;
  pp.part_ml = part_ml;
  const int* m = plan + 5 * (size_t)entries;
  pp.merge_first = m;
  pp.merge_count = m + merges;
  pp.merge_slot = m + 2 * (size_t)merges;
  pp.merge_parts = m + 3 * (size_t)merges;
  pp.merges = merges;
  return prefill_dispatch(q, q_stride, kc, vc, block_table, table_width, plan, plan + entries, entries, rows_per_tile,
                          token_row, pos, out, Hq, Hkv, D, page_size, scale, 0, pp, st);
}
