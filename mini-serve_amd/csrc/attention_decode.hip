// Decode attention for bfloat16: one query token per sequence over the paged cache, split over the
// keys so that a small batch still fills the chip, then a fixed-order reduction of the splits.
//
// Cache layouts (one KV head of one page is contiguous):
//   keys   K [pages, Hkv, page_size = 16, D]     a token's head is a row of D
//   values V [pages, Hkv, D, page_size = 16]     transposed within the page: the 16 tokens of one
//                                                head element are contiguous
// Both feed v_mfma_f32_16x16x32_bf16 straight from global memory with one vector load per lane:
//   scores  S^T[token, query] : A operand = K rows (i = token), B operand = Q (j = query head of the group)
//   output  O^T[d, query]     : A operand = V^T (i = d, k = token), B operand = P (j = query, k = token)
// The two score products of a 32-token chunk take their key rows in an order chosen so that a lane
// of the results holds 8 consecutive tokens of one page for one query (lane group g: page g / 2 of
// the chunk, tokens 8 (g % 2) .. + 7; four from each product). The MFMA's k index of the second
// product is mapped to tokens in the same way, so exactly these 8 values are the lane's P operand
// (probabilities never move between lanes) and its V^T operand is one 16-byte load.
//
// Grid: (rows * Hkv, splits). A block of 4 waves takes a contiguous range of 32-token chunks; its
// waves take a quarter of them each and are merged in LDS. splits == 1 writes the result directly.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define PAGE 16
#define CHUNK 32  // tokens per step of a wave: two pages

// Keys and values of one 32-token chunk as a wave holds them: the matrix operands themselves.
template <int D>
struct DecodeTile {
  bf16x8 ka[D / 32], kb[D / 32];
  bf16x8 v[D / 16];
};

// The fused form takes, instead of finished queries and a cache that already holds the new token, the
// qkv projection as it leaves the small-M product: float partial sums [splits, tokens, (Hq + 2 Hkv) D].
// Every wave sums, norms and rotates the queries of its KV head's group itself (up to 256 floats; the
// block's waves share the work if there are more);
// the one wave whose chunks end with the sequence's last token does the same for the new key, takes
// the new value, stores both into the cache and puts them into its operands of that chunk in
// registers (what its loads brought from the not yet written slot is replaced, so no store has to be
// waited for). This is the work of the QK-norm / rotation / store kernel, which a step of single
// tokens then does not launch.
struct FusedQkv {
  const float* parts;      // [splits, tokens, row_width]
  int splits;
  long long split_stride;  // floats between splits
  int row_width;           // (Hq + 2 Hkv) D
  const bf16* q_weight;    // [D] each, or both nullptr: no norm
  const bf16* k_weight;
  float eps;
  const float* rope;       // [tokens, D]: cosines, then sines, of D / 2 angles; nullptr: no rotation
  int store;               // 0: another layer owns the cache, the new token is already in it
};

// Four consecutive elements d0 .. d0 + 3 of a head whose D / 4 holders are neighbouring lanes (an
// aligned group): RMSNorm over the head with weight w (if any), then rotation by the angles of
// `rope_row` (if any), element d paired with d +- D / 2. Every lane of the wave must call this.
template <int D>
__device__ __forceinline__ void head_norm_rotate(float (&x)[4], int d0, const bf16* __restrict__ w, float eps,
                                                 const float* __restrict__ rope_row) {
  if (w != nullptr) {
    float ss = x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
#pragma unroll
    for (int o = 1; o < D / 4; o <<= 1) ss += __shfl_xor(ss, o, WAVE);
    const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = x[e] * rstd * to_f32(w[d0 + e]);
  }
  if (rope_row != nullptr) {
    const int j0 = d0 % (D / 2);
    const float4 c = *reinterpret_cast<const float4*>(rope_row + j0);
    const float4 sn = *reinterpret_cast<const float4*>(rope_row + D / 2 + j0);
    const float cs[4] = {c.x, c.y, c.z, c.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
    const bool low = d0 < D / 2;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float partner = __shfl_xor(x[e], D / 8, WAVE);
      x[e] = low ? x[e] * cs[e] - partner * ss[e] : x[e] * cs[e] + partner * ss[e];
    }
  }
}

// Sum over the splits, in ascending order, of four floats at `at` of each split.
__device__ __forceinline__ void sum_parts4(float (&x)[4], const float* __restrict__ parts, int splits, long long stride, size_t at) {
  x[0] = x[1] = x[2] = x[3] = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 4) {  // the loads of four splits go out together
    float4 a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      a[u] = *reinterpret_cast<const float4*>(parts + (size_t)(s0 + u < splits ? s0 + u : 0) * stride + at);
      if (s0 + u >= splits) a[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      x[0] += a[u].x; x[1] += a[u].y; x[2] += a[u].z; x[3] += a[u].w;
    }
  }
}

template <int D, bool FUSED>
__global__ __launch_bounds__(256, 2) void attn_decode_split_kernel(
    const bf16* __restrict__ q, int q_stride, bf16* kc_rw, bf16* vc_rw,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ tokens,
    const int* __restrict__ token_row, const int* __restrict__ pos, bf16* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, int Hq, int Hkv, float scale, int window, FusedQkv fin) {
  constexpr int KK = D / 32;  // k-steps of the score product
  constexpr int DB = D / 16;  // 16-wide blocks of the head
  const bf16* kc = kc_rw;
  const bf16* vc = vc_rw;
  const int G = Hq / Hkv;
  const int b = blockIdx.x / Hkv, kvh = blockIdx.x % Hkv;
  const int split = blockIdx.y, splits = gridDim.y;
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  const int tok = tokens ? tokens[b] : b;
  const int kv_len = pos[tok] + 1;
  const int lo = (window > 0 && kv_len > window) ? kv_len - window : 0;
  const int lo_al = lo & ~(CHUNK - 1);
  const int n_chunks = (kv_len - lo_al + CHUNK - 1) / CHUNK;
  const int per = (n_chunks + splits - 1) / splits;
  const int c_begin = split * per;
  const int c_end = min(n_chunks, c_begin + per);
  const int* table = block_table + (size_t)token_row[tok] * table_width;

  // Query operand: column r is query head kvh * G + r of the group (zero beyond the group).
  bf16x8 qf[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    if (!FUSED && r < G) {
      qf[kk] = *reinterpret_cast<const bf16x8*>(q + (size_t)tok * q_stride + (size_t)(kvh * G + r) * D + kk * 32 + g * 8);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[kk][i] = static_cast<bf16>(0.f);
    }
  }

  // Scores are kept in units of log2 (exp2 is one instruction); maxima, also those handed to the
  // reduction kernel, are in the same units.
  const float scale2 = scale * 1.44269504088896340736f;
  float m_run = -INFINITY, l_run = 0.f;  // of query r (replicated over the four lane groups)
  floatx4 o[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) o[i] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Two chunks are in flight per wave: while one is multiplied the next one's keys and values are
  // already on their way, and the page ids of the one after that. Loads go out in chunk order, so
  // one pair of prefetched page ids is enough.
  // A wave takes a contiguous quarter of the block's chunks (not every fourth chunk): with a request's
  // pages next to each other in memory, waves that step through every fourth chunk in lockstep keep
  // hitting the same few memory channels (measured on the address pattern alone: 5.1 -> 5.8 TB/s).
  const int per_wave = (c_end - c_begin + 3) / 4;
  const int w_begin = c_begin + wave * per_wave, w_end = min(c_end, w_begin + per_wave);
  // Fused form: this wave's chunks end with the sequence's last one, which holds the new token.
  const bool has_new = FUSED && fin.store && w_begin < w_end && w_end == n_chunks;
  __shared__ __attribute__((aligned(16))) bf16 qs[FUSED ? 4 : 1][FUSED ? 16 * D : 8];  // each wave's queries [G, D]
  __shared__ __attribute__((aligned(16))) bf16 kv_new[FUSED ? 2 * D : 8];              // the new key, then the new value
  // The two table entries of a chunk are fetched together and without a condition (one 8-byte load where
  // the table allows it; past the wave's last chunk that chunk's again, dropped): a load that waits for
  // the outcome of another costs a round trip each, before the first key is even asked for. Whether the
  // chunk has a second page at all is settled when the entries are used.
  const bool pair_ids = (table_width % 2 == 0) && (reinterpret_cast<size_t>(block_table) % 8 == 0);
  int p0n = 0, p1n = 0;
  auto fetch_ids = [&](int c) {
    const int idx = (lo_al + min(c, w_end - 1) * CHUNK) / PAGE;  // even: a chunk is two pages
    if (pair_ids) {
      const int2 v = *reinterpret_cast<const int2*>(table + idx);
      p0n = v.x;
      p1n = v.y;
    } else {
      p0n = table[idx];
      p1n = table[min(idx + 1, table_width - 1)];
    }
  };
  auto load = [&](DecodeTile<D>& t, int c) {
    const int p0 = max(p0n, 0);  // a page behind the window was given back: its tokens are masked below
    const int p1 = (lo_al + c * CHUNK + PAGE < kv_len) ? max(p1n, 0) : p0;
    fetch_ids(c + 1);
    // Key rows: lane r feeds row r of both products. Product a takes tokens 0-3 and 8-11 of each page,
    // product b tokens 4-7 and 12-15 (rows 0-7 from the chunk's first page, 8-15 from its second).
    const int kp = r < 8 ? p0 : p1;
    const int kt = (r % 4) + 8 * ((r / 4) % 2);
    const bf16* k0 = kc + (((size_t)kp * Hkv + kvh) * PAGE + kt) * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      t.ka[kk] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(k0 + kk * 32));
      t.kb[kk] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(k0 + 4 * D + kk * 32));
    }
    // V^T operand: element d = db * 16 + r, tokens 8 (g % 2) .. + 7 of page g / 2.
    const bf16* v0 = vc + (((size_t)(g < 2 ? p0 : p1) * Hkv + kvh) * D + r) * PAGE + (g % 2) * 8;
#pragma unroll
    for (int db = 0; db < DB; ++db) t.v[db] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(v0 + (size_t)db * 16 * PAGE));
  };
  auto multiply = [&](DecodeTile<D>& t, int c) {
    const int t0 = lo_al + c * CHUNK;
    if (FUSED && has_new && c == n_chunks - 1) {
      // The new token is token j of this chunk: key row jt of page jp, that is row r_new of product a
      // or b; and element j % 8 of the value operands of lane group 2 jp + jt / 8.
      const int j = kv_len - 1 - t0, jp = j / PAGE, jt = j % PAGE;
      const int r_new = jp * 8 + (jt / 8) * 4 + jt % 4;
      const bool second = (jt / 4) & 1;
      if (r == r_new) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const bf16x8 kn = *reinterpret_cast<const bf16x8*>(&kv_new[kk * 32 + g * 8]);
          if (second) t.kb[kk] = kn;
          else t.ka[kk] = kn;
        }
      }
      // A chunk that ends in its first page reads that page for its second half as well (masked, but a
      // probability of 0 does not wipe out whatever the unwritten slot happens to hold).
      const bool twice = t0 + PAGE >= kv_len;
      if (g % 2 == jt / 8 && (g / 2 == jp || twice)) {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const bf16 vn = kv_new[D + db * 16 + r];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e == jt % 8) t.v[db][e] = vn;
        }
      }
    }
    floatx4 s0 = floatx4{0.f, 0.f, 0.f, 0.f}, s1 = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.ka[kk], qf[kk], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.kb[kk], qf[kk], s1, 0, 0, 0);
    }
    // This lane: tokens tl + i (s0) and tl + 4 + i (s1) of query r, tl = t0 + 16 (g / 2) + 8 (g % 2).
    const int tl = t0 + 8 * g;
    float sc[8];
    float m_new = m_run;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ta = tl + i, tb = ta + 4;
      sc[i] = (ta >= lo && ta < kv_len) ? s0[i] * scale2 : -INFINITY;
      sc[4 + i] = (tb >= lo && tb < kv_len) ? s1[i] * scale2 : -INFINITY;
      m_new = fmaxf(m_new, fmaxf(sc[i], sc[4 + i]));
    }
    m_new = rows4_max(m_new);
    // A chunk that holds no visible token at all cannot occur: chunks start at the window's first
    // token's chunk and end at the last token's.
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = __builtin_amdgcn_exp2f(sc[i] - m_new);
      psum += p;
      pf[i] = static_cast<bf16>(p);
    }
    psum = rows4_sum(psum);
    const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
    l_run = l_run * corr + psum;
    m_run = m_new;
    // O^T[d, query]: a lane's output values are all of its own query r.
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[db][i] *= corr;
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.v[db], pf, o[db], 0, 0, 0);
    }
  };
  {
    DecodeTile<D> ta, tb;
    int c = w_begin;
    if (c < w_end) {
      fetch_ids(c);
      load(ta, c);
    }
    if (FUSED) {
      // Queries of the group: G * D floats, four per lane and round. (The first chunk is on its way.)
      const size_t row = (size_t)tok * fin.row_width;
      const float* rope_row = fin.rope ? fin.rope + (size_t)tok * D : nullptr;
      const int gd = G * D;
      // The wave that holds the new token asks for its key (lanes 0 .. D / 4 - 1) and value (lanes 32 ..
      // 32 + D / 4 - 1) first, so that they arrive while the queries are worked on.
      const bool is_k = lane < 32, kv_valid = lane % 32 < D / 4;
      const int kv_d0 = kv_valid ? (lane % 32) * 4 : 0;
      float xn[4] = {0.f, 0.f, 0.f, 0.f};
      if (has_new) sum_parts4(xn, fin.parts, fin.splits, fin.split_stride, row + (size_t)(is_k ? Hq + kvh : Hq + Hkv + kvh) * D + kv_d0);
      // Up to 256 floats (a lane's four of one round): every wave works its own copy out, no barrier.
      // More: the block's waves share the work (a wave takes whole heads) and meet once.
      const bool together = gd > 4 * WAVE;
      const int step = together ? 4 * 256 : 4 * WAVE;
      bf16* q_lds = together ? &qs[0][0] : &qs[wave][0];
      for (int base = 0; base < gd; base += step) {
        const int e0 = base + (together ? tid : lane) * 4;
        const bool valid = e0 < gd;
        const int ec = valid ? e0 : 0;
        float x[4];
        sum_parts4(x, fin.parts, fin.splits, fin.split_stride, row + (size_t)kvh * gd + ec);
        head_norm_rotate<D>(x, ec % D, fin.q_weight, fin.eps, rope_row);
        if (valid) {
          bf16x4 xb;
#pragma unroll
          for (int e = 0; e < 4; ++e) xb[e] = static_cast<bf16>(x[e]);
          *reinterpret_cast<bf16x4*>(q_lds + ec) = xb;
        }
      }
      if (together) __syncthreads();
      if (r < G) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[kk] = *reinterpret_cast<const bf16x8*>(q_lds + r * D + kk * 32 + g * 8);
      }
      if (has_new) {
        // The new key and value: into the cache, and into LDS for this wave's last chunk.
        float xk[4] = {xn[0], xn[1], xn[2], xn[3]};
        head_norm_rotate<D>(xk, kv_d0, fin.k_weight, fin.eps, rope_row);
        const int p = kv_len - 1;
        const size_t page = (size_t)table[p / PAGE];
        if (kv_valid && is_k) {
          bf16x4 xb;
#pragma unroll
          for (int e = 0; e < 4; ++e) xb[e] = static_cast<bf16>(xk[e]);
          *reinterpret_cast<bf16x4*>(&kv_new[kv_d0]) = xb;
          *reinterpret_cast<bf16x4*>(kc_rw + ((page * Hkv + kvh) * PAGE + p % PAGE) * D + kv_d0) = xb;
        }
        if (kv_valid && !is_k) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bf16 vb = static_cast<bf16>(xn[e]);
            kv_new[D + kv_d0 + e] = vb;
            vc_rw[((page * Hkv + kvh) * D + kv_d0 + e) * PAGE + p % PAGE] = vb;
          }
        }
      }
    }
    while (c < w_end) {
      if (c + 1 < w_end) load(tb, c + 1);
      multiply(ta, c);
      c += 1;
      if (c >= w_end) break;
      if (c + 1 < w_end) load(ta, c + 1);
      multiply(tb, c);
      c += 1;
    }
  }

  // Merge the block's four waves: per query (m, l) and O[query][D].
  __shared__ float sm[4][16], sl[4][16];
  __shared__ float so[4][16][D + 1];
  if (g == 0) {
    sm[wave][r] = m_run;
    sl[wave][r] = l_run;
  }
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i) so[wave][r][db * 16 + 4 * g + i] = o[db][i];
  __syncthreads();
  for (int e = tid; e < G * D; e += 256) {
    const int qh = e / D, d = e % D;
    float M = fmaxf(fmaxf(sm[0][qh], sm[1][qh]), fmaxf(sm[2][qh], sm[3][qh]));
    float L = 0.f, O = 0.f;
    if (M > -INFINITY) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float f = __builtin_amdgcn_exp2f(sm[w][qh] - M);  // 0 for a wave that saw nothing
        L += sl[w][qh] * f;
        O += so[w][qh][d] * f;
      }
    }
    const int head = kvh * G + qh;
    if (splits == 1) {
      out[((size_t)tok * Hq + head) * D + d] = static_cast<bf16>(O / L);
    } else {
      const size_t at = ((size_t)b * Hq + head) * splits + split;
      part_o[at * D + d] = O;
      if (d == 0) {
        part_ml[at * 2] = M;
        part_ml[at * 2 + 1] = L;
      }
    }
  }
}

// Reduction of the splits in ascending order: grid (rows, Hq), D threads. Loads go out 32 splits at
// a time (all of them, for most shapes), so that their latencies overlap; the order of the sums is
// the order of the splits whatever the batching.
template <int D>
__global__ __launch_bounds__(D) void attn_decode_reduce_kernel(const float* __restrict__ part_o,
                                                                const float* __restrict__ part_ml,
                                                                const int* __restrict__ tokens, bf16* __restrict__ out,
                                                                int Hq, int splits) {
  constexpr int NB = 32;
  const int b = blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  const size_t base = ((size_t)b * Hq + head) * splits;
  const float2* ml = reinterpret_cast<const float2*>(part_ml) + base;
  float M = -INFINITY, L = 0.f, O = 0.f;
  if (splits <= NB) {
    // One round: everything is asked for before the maximum is known.
    float2 q[NB];
    float o[NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const bool in = u < splits;
      q[u] = in ? ml[u] : make_float2(-INFINITY, 0.f);
      o[u] = in ? part_o[(base + u) * D + d] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) M = fmaxf(M, q[u].x);
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const float f = q[u].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(q[u].x - M);  // an empty or absent split adds nothing
      L += q[u].y * f;
      O += o[u] * f;
    }
  } else {
    for (int s0 = 0; s0 < splits; s0 += NB) {
      float m[NB];
#pragma unroll
      for (int u = 0; u < NB; ++u) m[u] = s0 + u < splits ? ml[s0 + u].x : -INFINITY;
#pragma unroll
      for (int u = 0; u < NB; ++u) M = fmaxf(M, m[u]);
    }
    for (int s0 = 0; s0 < splits; s0 += NB) {
      float2 q[NB];
      float o[NB];
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const bool in = s0 + u < splits;
        q[u] = in ? ml[s0 + u] : make_float2(-INFINITY, 0.f);
        o[u] = in ? part_o[(base + s0 + u) * D + d] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const float f = q[u].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(q[u].x - M);
        L += q[u].y * f;
        O += o[u] * f;
      }
    }
  }
  const int tok = tokens ? tokens[b] : b;
  out[((size_t)tok * Hq + head) * D + d] = static_cast<bf16>(O / L);
}

// rows decode tokens (tokens[i] = flat token index, or nullptr for the identity). part_o holds
// rows * Hq * splits * D floats, part_ml rows * Hq * splits * 2 (unused when splits == 1).
template <bool FUSED>
static int launch_decode(const bf16* q, int q_stride, bf16* kc, bf16* vc, const int* block_table, int table_width,
                         const int* tokens, const int* token_row, const int* pos, bf16* out, float* part_o, float* part_ml,
                         int rows, int splits, int Hq, int Hkv, int D, float scale, int window, FusedQkv fin, hipStream_t st,
                         bool reduce = true) {
  dim3 grid(rows * Hkv, splits);
#define LAUNCH(DD)                                                                                                      \
  attn_decode_split_kernel<DD, FUSED><<<grid, 256, 0, st>>>(q, q_stride, kc, vc, block_table, table_width, tokens,      \
                                                            token_row, pos, out, part_o, part_ml, Hq, Hkv, scale,       \
                                                            window, fin);                                               \
  if (splits > 1 && reduce) attn_decode_reduce_kernel<DD><<<dim3(rows, Hq), DD, 0, st>>>(part_o, part_ml, tokens, out, Hq, splits)
  if (D == 128) { LAUNCH(128); } else { LAUNCH(64); }
#undef LAUNCH
  return launch_status();
}

extern "C" int ms_attention_decode_bf16(const void* q, int q_stride, const void* kc, const void* vc,
                                        const int* block_table, int table_width, const int* tokens,
                                        const int* token_row, const int* pos, void* out, float* part_o, float* part_ml,
                                        int rows, int splits, int Hq, int Hkv, int D, int page_size, float scale,
                                        int window, hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (page_size != PAGE || (D != 64 && D != 128)) return MS_UNSUPPORTED;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hq / Hkv > 16 || splits < 1 || splits > 65535 || window < 0 || table_width <= 0 ||
      q_stride < Hq * D || q_stride % 8 || (splits > 1 && (!part_o || !part_ml)))
    return MS_BAD_ARG;
  return launch_decode<false>((const bf16*)q, q_stride, (bf16*)kc, (bf16*)vc, block_table, table_width, tokens, token_row,
                              pos, (bf16*)out, part_o, part_ml, rows, splits, Hq, Hkv, D, scale, window, FusedQkv{}, st);
}

// The same over the qkv projection's partial sums `parts` [qkv_splits, tokens, (Hq + 2 Hkv) D] (floats,
// qkv_split_stride apart) of a step whose rows bring one token each: per-head RMSNorm of q and k with
// bfloat16 weights [D] (both nullptr: none), rotation over the whole head by the table `rope`
// [tokens, D] (nullptr: none) in pairs (j, j + D/2) (rope_pairing must be MS_ROPE_HALVES: the kernel's lanes
// hold the halves of a head side by side; any other pairing is MS_UNSUPPORTED), and, with store != 0, the new token's key and value written to its place
// in the cache (its page is taken from the block table at pos).
extern "C" int ms_attention_decode_fused_bf16(const float* parts, int qkv_splits, long long qkv_split_stride,
                                              const void* q_weight, const void* k_weight, float eps, const float* rope,
                                              int rope_pairing, int store, void* kc, void* vc, const int* block_table, int table_width,
                                              const int* tokens, const int* token_row, const int* pos, void* out,
                                              float* part_o, float* part_ml, int rows, int splits, int Hq, int Hkv, int D,
                                              int page_size, float scale, int window, int reduce, hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (page_size != PAGE || (D != 64 && D != 128) || (rope != nullptr && rope_pairing != MS_ROPE_HALVES)) return MS_UNSUPPORTED;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hq / Hkv > 16 || splits < 1 || splits > 65535 || window < 0 || table_width <= 0 ||
      (splits > 1 && (!part_o || !part_ml)) || (splits > 1 && reduce && out == nullptr) || (splits == 1 && out == nullptr) ||
      parts == nullptr || qkv_splits < 1 || qkv_split_stride % 4 ||
      (q_weight == nullptr) != (k_weight == nullptr))
    return MS_BAD_ARG;
  FusedQkv fin;
  fin.parts = parts;
  fin.splits = qkv_splits;
  fin.split_stride = qkv_split_stride;
  fin.row_width = (Hq + 2 * Hkv) * D;
  fin.q_weight = (const bf16*)q_weight;
  fin.k_weight = (const bf16*)k_weight;
  fin.eps = eps;
  fin.rope = rope;
  fin.store = store;
  return launch_decode<true>(nullptr, 0, (bf16*)kc, (bf16*)vc, block_table, table_width, tokens, token_row, pos, (bf16*)out,
                             part_o, part_ml, rows, splits, Hq, Hkv, D, scale, window, fin, st, reduce != 0);
}

// ---------------------------------------------------------------------------------------------
// The reduction of the splits and the output projection in one kernel, for up to 16 rows that bring one
// token each: Y[m, n] = sum over heads h, d of out[m, h, d] W[n, h D + d], out being what the reduction
// kernel above would have written. A block owns HB heads (a slice of K) and NW * 16 rows of W, one wave
// per 16 rows. Its waves first ask for their weights, then merge the splits of the block's heads for every
// row (a wave per (row, head): a lane per split finds the maximum and the weights by wave reductions;
// then every thread sums its elements over the splits in ascending order), leave the merged rows in LDS
// as bfloat16, and multiply. K is split over the grid by heads: block column c writes the float partial
// sums P[c, m, n], which the reader of the residual stream adds up as it does for the other products
// of few rows. At most 64 splits (a lane each).
#define MERGE_MAX_SPLITS 64
#define MERGE_MAX_HB 4
// HB heads per block; every wave takes NPW blocks of 16 rows of W (so that a wide W does not mean many
// blocks that each merge the same splits again).
template <int D, int HB, int NPW>
__global__ __launch_bounds__(256) void attn_merge_project_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 const bf16* __restrict__ W, float* __restrict__ P, int rows,
                                                                 int Hq, int splits, int N) {
  constexpr int NW = 4, KB = HB * D, STEPS = KB / 64;
  __shared__ float fw[HB][16][MERGE_MAX_SPLITS];                 // weight of split s in row m of head j
  __shared__ __attribute__((aligned(16))) bf16 xs[16][KB + 8];   // merged rows; rows beyond `rows` are zero
  __shared__ float4 psum[NW * WAVE];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  const int h0 = blockIdx.x * HB;  // first head of this block
  const int K = Hq * D;            // columns of W
  const int nb0 = (blockIdx.y * NW + wave) * NPW * 16;
  // weights first: they come from memory, everything below from the cache
  union Chunk { uint4 u; bf16x8 v; };
  Chunk a[NPW][STEPS][2];
#pragma unroll
  for (int q = 0; q < NPW; ++q) {
    const bf16* wp = W + (size_t)min(nb0 + q * 16 + r, N - 1) * K + (size_t)h0 * D + g * 16;
#pragma unroll
    for (int u = 0; u < STEPS; ++u) {
      a[q][u][0].u = *reinterpret_cast<const uint4*>(wp + u * 64);
      a[q][u][1].u = *reinterpret_cast<const uint4*>(wp + u * 64 + 8);
    }
  }
  for (int e = tid; e < 16 * (KB / 4); e += NW * WAVE)  // rows beyond `rows` read as zero
    *reinterpret_cast<uint2*>(&xs[e / (KB / 4)][(e % (KB / 4)) * 4]) = make_uint2(0, 0);
  // the weights of the splits: wave w takes the (row, head) pairs w, w + NW, ...
  for (int p = wave; p < rows * HB; p += NW) {
    const int m = p / HB, j = p % HB;
    const float2* ml = reinterpret_cast<const float2*>(part_ml) + ((size_t)m * Hq + h0 + j) * splits;
    const float2 q = lane < splits ? ml[lane] : make_float2(-INFINITY, 0.f);
    const float mx = wave_max(q.x);
    const float f = q.x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(q.x - mx);  // an empty or absent split adds nothing
    const float total = wave_sum(q.y * f);
    fw[j][m][lane] = f / total;
  }
  __syncthreads();
  // Merged rows. An element is four consecutive d of one (row, head); there are E = rows * HB * D / 4 of
  // them. With fewer elements than threads the splits of an element are shared out among SG threads
  // (contiguous ranges, each summed in ascending order, the ranges then added in ascending order), so
  // that one row's 64 splits are not one thread's 64 dependent loads.
  const int E = rows * HB * (D / 4);
  const int threads = NW * WAVE;
  const int SG = E >= threads ? 1 : threads / E;
  const int per = (splits + SG - 1) / SG;
  for (int base = 0; base < E * SG; base += threads) {
    const int item = base + tid;
    const bool live = item < E * SG;
    const int e = live ? item % E : 0, sg = live ? item / E : 0;
    const int m = e / (HB * (D / 4)), c = e % (HB * (D / 4));
    const int j = c / (D / 4), d = (c % (D / 4)) * 4;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    const int s_end = min(splits, (sg + 1) * per);
    if (live) {
      const float* po = part_o + (((size_t)m * Hq + h0 + j) * splits) * D + d;
      for (int s0 = sg * per; s0 < s_end; s0 += 8) {
        float4 t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = *reinterpret_cast<const float4*>(po + (size_t)min(s0 + u, splits - 1) * D);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const float f = s0 + u < s_end ? fw[j][m][s0 + u] : 0.f;
          acc.x += t[u].x * f; acc.y += t[u].y * f; acc.z += t[u].z * f; acc.w += t[u].w * f;
        }
      }
    }
    if (SG > 1) {  // then E * SG <= threads: one round
      psum[tid] = acc;
      __syncthreads();
      if (tid < E) {
        acc = psum[tid];
        for (int q = 1; q < SG; ++q) {
          const float4 t = psum[q * E + tid];
          acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
        }
      }
    }
    if (live && sg == 0) {
      union { uint2 u; bf16 b[4]; } o;
      o.b[0] = static_cast<bf16>(acc.x); o.b[1] = static_cast<bf16>(acc.y);
      o.b[2] = static_cast<bf16>(acc.z); o.b[3] = static_cast<bf16>(acc.w);
      *reinterpret_cast<uint2*>(&xs[m][j * D + d]) = o.u;
    }
  }
  __syncthreads();
  bf16x8 x[STEPS][2];
#pragma unroll
  for (int u = 0; u < STEPS; ++u) {
    const bf16* xp = &xs[r][u * 64 + g * 16];
    x[u][0] = *reinterpret_cast<const bf16x8*>(xp);
    x[u][1] = *reinterpret_cast<const bf16x8*>(xp + 8);
  }
#pragma unroll
  for (int q = 0; q < NPW; ++q) {
    floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < STEPS; ++u) {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[q][u][0].v, x[u][0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[q][u][1].v, x[u][1], acc, 0, 0, 0);
    }
    // acc[e] = Y[m = r][n = nb + 4 g + e] of this block's heads
    const int nb = nb0 + q * 16;
    if (r < rows && nb + 16 <= N)
      *reinterpret_cast<float4*>(P + ((size_t)blockIdx.x * rows + r) * N + nb + 4 * g) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  }
}

// Heads per block so that the output projection's partial sums number at most 16: 1, 2, 3 or 4 (a block's
// slice of K, HB * D, is then a whole number of 64-element steps for both head sizes).
static int merge_project_heads_per_block(int Hq) {
  const int hb = (Hq + 15) / 16;
  return hb < 1 || hb > MERGE_MAX_HB || Hq % hb ? 0 : hb;
}

// How many partial sums ms_attention_merge_project leaves for this shape, or -1 where it has no kernel and
// the reduction kernel and the output projection must run apart. The one place that decides it: the launch
// below asks the same function, so a caller that sizes its buffers by the answer is never refused afterwards.
extern "C" int ms_attention_merge_project_splits(int rows, int Hq, int D, int splits, int N) {
  const int hb = merge_project_heads_per_block(Hq);
  if (hb == 0 || rows < 1 || rows > 16 || splits < 1 || splits > MERGE_MAX_SPLITS || (D != 64 && D != 128) || N <= 0 || N % 64)
    return -1;
  return Hq / hb;
}

// P [ms_attention_merge_project_splits(...), rows, N] (float partial sums) from the split attention's
// partial results of `rows` <= 16 single-token rows (part_o, part_ml as the decode kernels leave them)
// and the output projection's weight W [N, Hq * D]. MS_UNSUPPORTED exactly where that function says -1.
// The widest instance (D 128, 4 heads, 256 rows of W per block) holds its 256 registers of weights in the
// vector registers and moves 68 values through the accumulation registers; nothing goes to scratch memory.
extern "C" int ms_attention_merge_project(const float* part_o, const float* part_ml, const void* W, float* P, int rows,
                                          int Hq, int D, int splits, int N, hipStream_t st) {
  if (rows <= 0 || N <= 0) return MS_OK;
  if (part_o == nullptr || part_ml == nullptr || W == nullptr || P == nullptr || Hq <= 0 || splits < 1) return MS_BAD_ARG;
  const int out_splits = ms_attention_merge_project_splits(rows, Hq, D, splits, N);
  if (out_splits < 1) return MS_UNSUPPORTED;
  const int hb = Hq / out_splits;
  // Rows of W per block: 64, or 256 where that still leaves a block for every CU.
  const int npw = (N % 256 == 0 && (long)out_splits * (N / 256) >= 256) ? 4 : 1;
  dim3 grid(out_splits, N / (64 * npw));
  const bf16* w = (const bf16*)W;
#define LAUNCH(DD, HB, NPW) attn_merge_project_kernel<DD, HB, NPW><<<grid, 256, 0, st>>>(part_o, part_ml, w, P, rows, Hq, splits, N)
#define LAUNCH_HB(DD, NPW)                                                                                              \
  if (hb == 1) LAUNCH(DD, 1, NPW);                                                                                      \
  else if (hb == 2) LAUNCH(DD, 2, NPW);                                                                                 \
  else if (hb == 3) LAUNCH(DD, 3, NPW);                                                                                 \
  else LAUNCH(DD, 4, NPW)
  if (D == 128 && npw == 4) { LAUNCH_HB(128, 4); }
  else if (D == 128) { LAUNCH_HB(128, 1); }
  else if (npw == 4) { LAUNCH_HB(64, 4); }
  else { LAUNCH_HB(64, 1); }
#undef LAUNCH_HB
#undef LAUNCH
  return launch_status();
}
