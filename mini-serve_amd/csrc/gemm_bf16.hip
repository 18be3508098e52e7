// bfloat16 matrix products C[M, N] = X[M, K] * W[N, K]^T on the gfx950 matrix cores
// (v_mfma_f32_16x16x32_bf16, float32 accumulation), in three shapes:
//
//  * tile kernel, slabs straight into LDS (prefill, M large, K a multiple of 64): 128 x 128 macro-tiles,
//                  K-slabs of 64 loaded by global_load_lds into a ring of two stages with a bank
//                  swizzle, one barrier per slab, two blocks per CU; 4 waves in a 2 x 2 grid of wave tiles.
//                  Its largest form, 256 x 256 with four wave tiles of 128 x 128, has its loop over K
//                  written in assembly (all 512 registers of a lane, fragment reads and loads placed
//                  between the products by hand) and one block per CU that takes tiles in turn.
//  * tile kernel, slabs through registers (any K and alignment, or few tiles): BM x BN macro-tiles
//                  staged through LDS in K-slabs of 64 with a register prefetch of the next slab.
//  * small-M kernel (decode, M <= 64): pure weight streaming. A wave owns 16 weight rows and a slice
//                  of K, with 32-byte loads per lane; K is split over the grid into partial sums.
//
// Operand roles: the weight rows are the MFMA's A operand (its row index i = n) and the activation
// rows the B operand (column index j = m), so a lane ends up with four consecutive n of one m and
// stores them as one vector.
//
// Layout of v_mfma_f32_16x16x32_bf16 (lane l, g = l / 16, r = l % 16):
//   A operand: 8 values A[i = r][k = 8 g .. 8 g + 7]     B operand: 8 values B[k = 8 g .. 8 g + 7][j = r]
//   result:    4 values D[i = 4 g + 0..3][j = r]
// Any permutation of k that is the same for both operands leaves the result unchanged; the small-M
// kernel uses that to let a lane load 16 consecutive k at once.
#include "common.h"

#include <utility>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union Chunk {  // 8 bf16 = 16 bytes
  uint4 u;
  bf16x8 v;
  bf16 e[8];
};

// 8 consecutive k of one row, zero where the row or k is out of range.
__device__ __forceinline__ Chunk load_chunk(const bf16* __restrict__ base, int row, int rows, int k, int K, size_t ld, bool vec) {
  Chunk c;
  if (row < rows && vec && k + 8 <= K) {
    c.u = *reinterpret_cast<const uint4*>(base + (size_t)row * ld + k);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) c.e[i] = (row < rows && k + i < K) ? base[(size_t)row * ld + k + i] : static_cast<bf16>(0.f);
  }
  return c;
}

// Store four consecutive n of row m. mode 0: bf16, 1: float, 2: float +=.
__device__ __forceinline__ void store4(void* __restrict__ C, int mode, int m, int n, int M, int N, int ldc, floatx4 a, bool vec_ok) {
  if (m >= M || n >= N) return;
  const size_t at = (size_t)m * ldc + n;
  if (vec_ok && n + 3 < N) {
    if (mode == 0) {
      union { uint2 u; bf16 e[4]; } o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o.e[i] = static_cast<bf16>(a[i]);
      *reinterpret_cast<uint2*>((bf16*)C + at) = o.u;
    } else if (mode == 1) {
      *reinterpret_cast<float4*>((float*)C + at) = make_float4(a[0], a[1], a[2], a[3]);
    } else {
      float4 c = *reinterpret_cast<float4*>((float*)C + at);
      c.x += a[0]; c.y += a[1]; c.z += a[2]; c.w += a[3];
      *reinterpret_cast<float4*>((float*)C + at) = c;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (n + i >= N) break;
      if (mode == 0) ((bf16*)C)[at + i] = static_cast<bf16>(a[i]);
      else if (mode == 1) ((float*)C)[at + i] = a[i];
      else ((float*)C)[at + i] += a[i];
    }
  }
}

// SiLU and tanh-GELU on the hardware's exp2 and reciprocal (about 1 ulp each, in float32): what they lose
// disappears in the rounding to bfloat16, and the library forms take some 35 instructions a value, which in
// the epilogue of the gated tile product was a tenth of the kernel's time.
__device__ __forceinline__ float activate_fast(float x, int act) {
  if (act == MS_ACT_GELU_TANH) {
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    const float t = 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(u * 2.885390081777927f));  // tanh(u)
    return 0.5f * x * (1.f + t);
  }
  return x * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// Four consecutive n of row m: the store of one accumulator fragment. MODE 0: bf16, 1: float, 2: float +=.
// INSIDE: the tile's columns lie within the matrix and a lane's four are aligned for one store, so only
// the row is tested (a ragged last row of tiles, which any token count makes, runs the same code as the rest:
// code that only a few blocks run is not in the instruction cache when they get there).
template <int MODE, bool INSIDE>
__device__ __forceinline__ void store_fragment(void* __restrict__ C, int m, int n, int M, int N, int ldc, floatx4 a, bool vec_ok) {
  if constexpr (!INSIDE) {
    store4(C, MODE, m, n, M, N, ldc, a, vec_ok);
  } else {
    if (m >= M) return;
    const size_t at = (size_t)m * ldc + n;
    if constexpr (MODE == 0) {
      union { uint2 u; bf16 e[4]; } o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o.e[i] = static_cast<bf16>(a[i]);
      *reinterpret_cast<uint2*>((bf16*)C + at) = o.u;
    } else if constexpr (MODE == 1) {
      *reinterpret_cast<float4*>((float*)C + at) = make_float4(a[0], a[1], a[2], a[3]);
    } else {
      float4 c = *reinterpret_cast<float4*>((float*)C + at);
      c.x += a[0]; c.y += a[1]; c.z += a[2]; c.w += a[3];
      *reinterpret_cast<float4*>((float*)C + at) = c;
    }
  }
}

// Gate and up fragments of the same four outputs (W holds alternating blocks of 16 gate rows and 16 up
// rows): out[m, col ..] = act(gate) * up, bf16 with row stride ldc; `half` = N / 2 columns.
template <int ACT, bool INSIDE>
__device__ __forceinline__ void store_gated(bf16* __restrict__ out, int m, int col, int M, int half, int ldc, floatx4 gate, floatx4 up) {
  if (m >= M || (!INSIDE && col >= half)) return;
  union { uint2 u; bf16 e[4]; } o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o.e[e] = static_cast<bf16>(activate_fast(gate[e], ACT) * up[e]);
  *reinterpret_cast<uint2*>(out + (size_t)m * ldc + col) = o.u;
}

// A wave tile's accumulators acc[i][j] (i: block of 16 n, j: block of 16 m) to memory. m, n: this lane's
// row and first column in fragment (0, 0). MODE as above (3 + activation: gated, C unused).
template <int MODE, bool INSIDE, int FN, int FM>
__device__ __forceinline__ void store_fragments(const floatx4 (&acc)[FN][FM], void* C, void* Cbase, int m, int n, int M, int N, int ldc,
                                                bool vec_store) {
  if constexpr (MODE >= 3) {
    const int g4 = n % 16;  // the lane's group of four columns
#pragma unroll
    for (int i = 0; i + 1 < FN; i += 2)
#pragma unroll
      for (int j = 0; j < FM; ++j)
        store_gated<MODE - 3, INSIDE>((bf16*)Cbase, m + j * 16, (n - g4 + i * 16) / 2 + g4, M, N / 2, ldc, acc[i][j], acc[i + 1][j]);
  } else {
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
      for (int j = 0; j < FM; ++j) store_fragment<MODE, INSIDE>(C, m + j * 16, n + i * 16, M, N, ldc, acc[i][j], vec_store);
  }
}

// The same into a tile image in LDS as bfloat16 (MODE 0, or 3 + activation: gated). at: this lane's place
// in fragment (0, 0); row_bytes: stride of the image's rows.
template <int MODE, int FN, int FM>
__device__ __forceinline__ void stage_fragments(const floatx4 (&acc)[FN][FM], unsigned char* at, int row_bytes) {
  union { uint2 u; bf16 e[4]; } o;
  if constexpr (MODE >= 3) {
#pragma unroll
    for (int i = 0; i + 1 < FN; i += 2)
#pragma unroll
      for (int j = 0; j < FM; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) o.e[e] = static_cast<bf16>(activate_fast(acc[i][j][e], MODE - 3) * acc[i + 1][j][e]);
        *reinterpret_cast<uint2*>(at + j * 16 * row_bytes + (i / 2) * 32) = o.u;
      }
  } else {
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
      for (int j = 0; j < FM; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) o.e[e] = static_cast<bf16>(acc[i][j][e]);
        *reinterpret_cast<uint2*>(at + j * 16 * row_bytes + i * 32) = o.u;
      }
  }
}

// ---------------------------------------------------------------------------------------------
// Tile kernel.
#define BK 64
#define LDS_STRIDE (BK + 8)  // bf16 elements per LDS row: 144 bytes, keeps 16-byte alignment

// blockIdx.z splits K into slices of k_per (a multiple of BK); slice z writes to C + z * c_split_stride
// elements (float partial sums, mode 1), so that matrices with few output tiles still fill the chip.
template <int BM, int BN>
__global__ __launch_bounds__(256, 2) void gemm_bf16_tile_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                                void* __restrict__ Cbase, int mode, int M, int N, int Kfull,
                                                                int ldx, int ldc, int k_per, size_t c_split_stride) {
  constexpr int WM = BM / 2, WN = BN / 2;      // wave tile
  constexpr int FM = WM / 16, FN = WN / 16;    // 16 x 16 fragments per wave tile
  constexpr int XCH = BM * (BK / 8) / 256;     // 16-byte chunks per thread per slab
  constexpr int WCH = BN * (BK / 8) / 256;
  __shared__ __attribute__((aligned(16))) bf16 xs[BM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16 ws[BN * LDS_STRIDE];

  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int wm = (wave / 2) * WM, wn = (wave % 2) * WN;
  const bool vecx = (Kfull % 8 == 0) && (ldx % 8 == 0), vecw = (Kfull % 8 == 0);
  const int k_lo = blockIdx.z * k_per;
  const int K = min(Kfull, k_lo + k_per);  // this slice ends here; chunks beyond it read as zeros
  void* C = mode == 1 ? (void*)((float*)Cbase + blockIdx.z * c_split_stride) : Cbase;

  floatx4 acc[FN][FM];
#pragma unroll
  for (int i = 0; i < FN; ++i)
#pragma unroll
    for (int j = 0; j < FM; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  Chunk xr[XCH], wr[WCH];
  // A tile that lies wholly inside both matrices loads its slabs without any test (all loads of a
  // slab go out back to back); edge tiles and the last, shorter slab take the checked loads.
  const bool interior = vecx && vecw && m0 + BM <= M && n0 + BN <= N;
  const bf16* xg = X + (size_t)(m0 + tid / (BK / 8)) * ldx + (tid % (BK / 8)) * 8;
  const bf16* wg = W + (size_t)(n0 + tid / (BK / 8)) * Kfull + (tid % (BK / 8)) * 8;
  auto fetch = [&](int k0) __attribute__((always_inline)) {
    if (interior && k0 + BK <= K) {
#pragma unroll
      for (int i = 0; i < XCH; ++i) xr[i].u = *reinterpret_cast<const uint4*>(xg + (size_t)i * (256 / (BK / 8)) * ldx + k0);
#pragma unroll
      for (int i = 0; i < WCH; ++i) wr[i].u = *reinterpret_cast<const uint4*>(wg + (size_t)i * (256 / (BK / 8)) * Kfull + k0);
      return;
    }
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int c = tid + i * 256;
      xr[i] = load_chunk(X, m0 + c / (BK / 8), M, k0 + (c % (BK / 8)) * 8, K, ldx, vecx);
    }
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
      const int c = tid + i * 256;
      wr[i] = load_chunk(W, n0 + c / (BK / 8), N, k0 + (c % (BK / 8)) * 8, K, Kfull, vecw);
    }
  };
  auto stash = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int c = tid + i * 256;
      *reinterpret_cast<uint4*>(&xs[(c / (BK / 8)) * LDS_STRIDE + (c % (BK / 8)) * 8]) = xr[i].u;
    }
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
      const int c = tid + i * 256;
      *reinterpret_cast<uint4*>(&ws[(c / (BK / 8)) * LDS_STRIDE + (c % (BK / 8)) * 8]) = wr[i].u;
    }
  };

  fetch(k_lo);
  stash();
  __syncthreads();
  for (int k0 = k_lo; k0 < K; k0 += BK) {
    const bool more = k0 + BK < K;
    if (more) fetch(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 32) {
      bf16x8 wf[FN], xf[FM];
#pragma unroll
      for (int i = 0; i < FN; ++i)
        wf[i] = *reinterpret_cast<const bf16x8*>(&ws[(wn + i * 16 + r) * LDS_STRIDE + kk + g * 8]);
#pragma unroll
      for (int j = 0; j < FM; ++j)
        xf[j] = *reinterpret_cast<const bf16x8*>(&xs[(wm + j * 16 + r) * LDS_STRIDE + kk + g * 8]);
#pragma unroll
      for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], xf[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
    if (more) {
      stash();
      __syncthreads();
    }
  }

  const bool vec_store = (ldc % 4 == 0);
#pragma unroll
  for (int i = 0; i < FN; ++i)
#pragma unroll
    for (int j = 0; j < FM; ++j)
      store4(C, mode, m0 + wm + j * 16 + r, n0 + wn + i * 16 + g * 4, M, N, ldc, acc[i][j], vec_store);
}

// ---------------------------------------------------------------------------------------------
// Tile kernel with slabs loaded straight into LDS (global_load_lds, 16 bytes per lane): no staging
// registers and no LDS store instructions, STAGES slabs of 64 k in a ring, one barrier per slab. A load
// instruction of a wave fills 1 KB of LDS in lane order, that is 8 rows of 128 bytes; which 16-byte
// chunk of its row a lane fetches is chosen so that chunk c of tile row R lands in slot
// c ^ ((R >> 1) & 7) of the row: fragment reads (16 rows, one chunk column) then touch every bank
// once. Rows beyond M or N are read from the last valid row (their results are never stored); K must
// be a multiple of 64 and rows 16-byte aligned, which the caller checks.

// Wait until at most N of this wave's vector-memory loads are in flight (expcnt and lgkmcnt are left alone).
template <int N>
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

struct TileId {
  int m, n, split;
};

// Tile `t` of a grid of rows x cols tiles: column tiles run fastest, then row tiles, inside bands of
// `band_cols` column tiles. The blocks that run together share a row of activations; the band bounds
// how much weight memory is live until all row tiles have used it, so that it stays in the last-level
// cache.
__device__ __forceinline__ void banded(int t, int rows, int cols, int band_cols, int& m, int& n) {
  const int band = t / (band_cols * rows), w = t % (band_cols * rows);
  const int width = min(band_cols, cols - band * band_cols);
  m = w / width;
  n = band * band_cols + w % width;
}

// Block `block` of a one-dimensional grid over splits x row tiles x column tiles. Blocks are handed to
// the eight XCDs in turn (block L to XCD L % 8), each with an L2 of its own. With xcd_rows == 0 the
// tiles are walked in banded order over the whole grid: band_cols being a multiple of eight, a weight
// tile column stays with one XCD, and every XCD reads all activations. With xcd_rows = 2, 4 or 8 (the
// caller has checked that the tile counts divide) the XCDs form a grid of xcd_rows x 8 / xcd_rows, each
// owning a rectangle of tiles that it walks in banded order: then an XCD reads only its share of the
// activations, which is what counts when the weight matrix is the smaller operand.
__device__ __forceinline__ TileId tile_of_block(int block, int blocks, int row_tiles, int col_tiles, int xcd_rows, int band_cols) {
  const int tiles = row_tiles * col_tiles;
  const int splits = blocks / tiles;
  TileId id;
  int t;
  if (row_tiles == 1 && splits > 1) {
    // One row of tiles with K split (a product bound by streaming its weights): the split index runs
    // fastest, so that neighbouring blocks read neighbouring k ranges of the same weight rows rather
    // than the same k range of rows that lie a power of two apart (2-3 % faster at 32 to 128 rows).
    id.split = block % splits;
    t = block / splits;
  } else {
    t = block % tiles;
    id.split = block / tiles;
  }
  if (xcd_rows == 0) {
    banded(t, row_tiles, col_tiles, band_cols, id.m, id.n);
    return id;
  }
  const int xcd_cols = 8 / xcd_rows;
  const int xcd = t % 8, slot = t / 8;
  const int sub_rows = row_tiles / xcd_rows, sub_cols = col_tiles / xcd_cols;
  banded(slot, sub_rows, sub_cols, band_cols, id.m, id.n);
  id.m += (xcd / xcd_cols) * sub_rows;
  id.n += (xcd % xcd_cols) * sub_cols;
  return id;
}

// WR x WC waves per block, each with a wave tile of BM / WR x BN / WC.
template <int BM, int BN, int KS, int STAGES, int BLOCKS_PER_CU, int WR = 2, int WC = 2>
__global__ __launch_bounds__(WR * WC * WAVE, BLOCKS_PER_CU) void gemm_bf16_dma_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                               void* __restrict__ Cbase, int mode, int M, int N, int Kfull,
                                                               int ldx, int ldc, int k_per, size_t c_split_stride, int xcd_rows,
                                                               int band_cols) {
  constexpr int NW = WR * WC;
  constexpr int WM = BM / WR, WN = BN / WC;
  constexpr int FM = WM / 16, FN = WN / 16;
  constexpr int ROW_BYTES = KS * 2;           // a tile row: KS k of bf16
  constexpr int CPR = KS / 8;                 // 16-byte chunks per row
  constexpr int RPI = 1024 / ROW_BYTES;       // rows a load instruction of a wave fills
  constexpr int XI = BM / (NW * RPI), WI = BN / (NW * RPI);  // load instructions per wave and slab
  static_assert(BM % (NW * RPI) == 0 && BN % (NW * RPI) == 0, "every wave loads whole instructions of both operands");
  constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];  // STAGES * STAGE_BYTES

  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  const TileId id = tile_of_block(blockIdx.x, gridDim.x, (M + BM - 1) / BM, (N + BN - 1) / BN, xcd_rows, band_cols);
  const int m0 = id.m * BM, n0 = id.n * BN;
  const int wm = (wave / WC) * WM, wn = (wave % WC) * WN;
  const int k_lo = id.split * k_per;
  const int K = min(Kfull, k_lo + k_per);
  const int slabs = (K - k_lo) / KS;
  void* C = mode == 1 ? (void*)((float*)Cbase + id.split * c_split_stride) : Cbase;

  // Load side: instruction j of this wave fills tile rows (wave * XI + j) * 8 .. + 7.
  const int lrow = lane / CPR, lslot = lane % CPR;
  const bf16* xsrc[XI];
  const bf16* wsrc[WI];
#pragma unroll
  for (int j = 0; j < XI; ++j) {
    const int R = (wave * XI + j) * RPI + lrow;
    xsrc[j] = X + (size_t)min(m0 + R, M - 1) * ldx + k_lo + ((lslot ^ ((R >> 1) & (CPR - 1))) * 8);
  }
#pragma unroll
  for (int j = 0; j < WI; ++j) {
    const int R = (wave * WI + j) * RPI + lrow;
    wsrc[j] = W + (size_t)min(n0 + R, N - 1) * Kfull + k_lo + ((lslot ^ ((R >> 1) & (CPR - 1))) * 8);
  }
  auto issue = [&](int slab) __attribute__((always_inline)) {
    unsigned char* stage = lds + (slab % STAGES) * STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < XI; ++j)
      __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(xsrc[j] + (size_t)slab * KS),
                                       (void __attribute__((address_space(3)))*)(stage + (wave * XI + j) * 1024),
                                       16, 0, 0);
#pragma unroll
    for (int j = 0; j < WI; ++j)
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)(wsrc[j] + (size_t)slab * KS),
          (void __attribute__((address_space(3)))*)(stage + BM * ROW_BYTES + (wave * WI + j) * 1024), 16, 0, 0);
  };

  floatx4 acc[FN][FM];
#pragma unroll
  for (int i = 0; i < FN; ++i)
#pragma unroll
    for (int j = 0; j < FM; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Read side: the rows of a fragment are base + r with base a multiple of 16, so the slot of chunk c
  // is c ^ (r >> 1) for every fragment.
  const int sw = (r >> 1) & (CPR - 1);
  const int x_off = (wm + r) * ROW_BYTES, w_off = BM * ROW_BYTES + (wn + r) * ROW_BYTES;

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < slabs) issue(s);
  for (int k = 0; k < slabs; ++k) {
    // Slab k must have landed; the STAGES - 2 slabs after it may stay in flight (near the end there
    // are fewer of them: then everything is waited for).
    if (k + STAGES - 2 < slabs) wait_loads<(XI + WI) * (STAGES - 2)>();
    else wait_loads<0>();
    __syncthreads();  // slab k has landed for every wave, and every wave is done with slab k - 1
    if (k + STAGES - 1 < slabs) issue(k + STAGES - 1);
    const unsigned char* stage = lds + (k % STAGES) * STAGE_BYTES;
    // All fragments of the slab are asked for before the first product (the scheduler is told not to
    // move them back down): the reads return in order, so each product waits only for its own
    // operands while the later reads are still on their way.
    constexpr int STEPS = CPR / 4;
    bf16x8 wf[STEPS][FN], xf[STEPS][FM];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int slot = ((t * 4 + g) ^ sw) * 16;  // chunk column 4 t + g
#pragma unroll
      for (int i = 0; i < FN; ++i) wf[t][i] = *reinterpret_cast<const bf16x8*>(stage + w_off + i * 16 * ROW_BYTES + slot);
#pragma unroll
      for (int j = 0; j < FM; ++j) xf[t][j] = *reinterpret_cast<const bf16x8*>(stage + x_off + j * 16 * ROW_BYTES + slot);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < STEPS; ++t)
#pragma unroll
      for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[t][i], xf[t][j], acc[i][j], 0, 0, 0);
  }

  // Epilogue. Modes 0 to 2 store the fragments as they are. Mode 3 + an MS_ACT_* number is the gated one:
  // W holds alternating blocks of 16 gate rows and 16 up rows, so fragments 2 p and 2 p + 1 of a lane are
  // gate and up of the same four outputs: out[m, n / 2 ...] = act(gate) * up, bf16 [M, N / 2] with row
  // stride ldc (wave tiles with an odd number of fragments are never launched in this mode). The mode is
  // told apart once, not per fragment, so that each mode's stores are one straight run of code: with the
  // test inside, a tile's epilogue jumped through a hundred kilobytes of code the instruction cache had
  // never seen, which took longer than ten slabs of products.
  const bool vec_store = (ldc % 4 == 0);
  const bool inside = n0 + BN <= N && vec_store;  // the columns; rows are tested where they are stored
  // bfloat16 outputs of a tile whose columns lie inside the matrix, rows 16-byte aligned, go through LDS
  // (the ring is free after the loop): a lane's four values of a row into a padded row of the tile
  // (conflict-free), then every thread takes 16 bytes of a row, so that store instructions write whole
  // 128-byte lines instead of 32-byte pieces of sixteen rows each, which cost the L2 four times the requests.
  constexpr int OUT_ROW = BN * 2 + 16, GATED_ROW = BN + 16;
  if (inside && ldc % 8 == 0 && (size_t)Cbase % 16 == 0 &&
      ((mode == 0 && BM * OUT_ROW <= STAGES * STAGE_BYTES) || (mode >= 3 && BM * GATED_ROW <= STAGES * STAGE_BYTES))) {
    __syncthreads();  // every wave has read the last slab's fragments
    const int row_bytes = mode == 0 ? OUT_ROW : GATED_ROW;
    static_assert(MS_ACT_COUNT == 2, "one case per activation below");
    if (mode == 0) stage_fragments<0, FN, FM>(acc, lds + (wm + r) * OUT_ROW + (wn + g * 4) * 2, OUT_ROW);
    else if (mode == 3) stage_fragments<3, FN, FM>(acc, lds + (wm + r) * GATED_ROW + (wn / 2 + g * 4) * 2, GATED_ROW);
    else stage_fragments<4, FN, FM>(acc, lds + (wm + r) * GATED_ROW + (wn / 2 + g * 4) * 2, GATED_ROW);
    __syncthreads();
    const int chunks = (row_bytes - 16) / 16;  // 16-byte chunks of an output row of the tile
    bf16* out = (bf16*)Cbase + (size_t)m0 * ldc + (mode == 0 ? n0 : n0 / 2);
    for (int c = tid; c < BM * chunks; c += NW * WAVE) {
      const int row = c / chunks, ch = c % chunks;
      if (m0 + row < M)
        *reinterpret_cast<uint4*>(out + (size_t)row * ldc + ch * 8) = *reinterpret_cast<const uint4*>(lds + row * row_bytes + ch * 16);
    }
    return;
  }
  const int m = m0 + wm + r, n = n0 + wn + g * 4;
  if (inside) {
    switch (mode) {
      case 0: store_fragments<0, true, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      case 1: store_fragments<1, true, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      case 2: store_fragments<2, true, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      case 3: store_fragments<3, true, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      default: store_fragments<4, true, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
    }
  } else {
    switch (mode) {
      case 0: store_fragments<0, false, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      case 1: store_fragments<1, false, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      case 2: store_fragments<2, false, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      case 3: store_fragments<3, false, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
      default: store_fragments<4, false, FN, FM>(acc, C, Cbase, m, n, M, N, ldc, vec_store); break;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// 256 x 256 tile with four waves, each with a wave tile of 128 x 128: 16 fragment reads for 64
// products (eight waves with wave tiles of 64 x 128, which the kernel above can be built with, read 12 for 32), so that fragment reads and the loads into LDS
// together keep the LDS busy three quarters of the time the products take instead of all of it. The 256
// accumulator registers of a lane are all the AGPRs there are, and one wave per SIMD has nobody to
// cover its waits, so registers and instruction order of the loop over K are written out: the loop is
// one assembly statement. Layout of LDS, swizzle and operand roles are those of the kernel above.
//   registers: a[4 (8 i + j) ..] accumulators of fragment (i = weight block, j = row block)
//              v[128 + 4 i ..], v[160 + 4 j ..]  fragment set A (even 32-k steps: weights, rows)
//              v[192 + 4 i ..], v[224 + 4 j ..]  fragment set B (odd steps)
//              v[96 .. 111] byte offsets of this lane's 16 loads of a slab (8 of rows, 8 of weights)
//              v[112 .. 115] LDS addresses of the fragment reads (weights step 0 / 1, rows step 0 / 1)
//              s[80:81], s[82:83] where the next slab to load begins (rows, weights); s84 LDS address of
//              this wave's part of the stage it loads into; s85 distance to the other stage (its sign
//              alternates); s86 slabs left
//   per slab:  step 0: products on set A, between them the reads of set B (same slab, second step);
//              wait for the next slab's loads, barrier (every wave has read all it needs of this slab);
//              step 1: products on set B, between them the reads of set A from the next slab and the
//              loads of the slab after next into this slab's stage.
// The slab count must be at least 2 (the caller checks); rows beyond M or N read the last valid row.
// Between the assembly statement and the reads of the accumulators after it the compiler must leave the
// AGPRs alone: it has no use for them here (no matrix builtins, 96 VGPRs of its own and nothing spilled:
// the kernel's scratch size is 0), and every statement names all of them as clobbered.
// One block per CU stays for the whole product and takes tiles in turn. Measured at 8192^3, sustained, at
// the socket's power limit: 1,500 TFLOP/s against 1,260 of that eight-wave tile and 1,620 of the vendor
// library; at 2,048 x 24,576 x 4,096 1,506 against 1,175 and 1,530.

// Accumulator fragment F of the wide tile's loop, out of the AGPRs.
template <int F>
__device__ __forceinline__ floatx4 wide_acc() {
  floatx4 v;
  asm volatile("v_accvgpr_read_b32 %0, a[%4]\n\tv_accvgpr_read_b32 %1, a[%4+1]\n\tv_accvgpr_read_b32 %2, a[%4+2]\n\tv_accvgpr_read_b32 %3, a[%4+3]"
               : "=v"(v[0]), "=v"(v[1]), "=v"(v[2]), "=v"(v[3])
               : "n"(F * 4));
  return v;
}

// Fragments (2 P, J) and (2 P + 1, J) of the wide tile. MODE 0 to 2: stored as they are; 3 + an MS_ACT_*
// number: as gate and up. m: this lane's row in row block 0; nb: the wave tile's first column; g: the
// lane's group of four columns.
template <int MODE, bool INSIDE, int P, int J>
__device__ __forceinline__ void wide_store(void* C, void* Cbase, int m, int nb, int g, int M, int N, int ldc, bool vec_store) {
  const floatx4 a = wide_acc<(2 * P) * 8 + J>(), b = wide_acc<(2 * P + 1) * 8 + J>();
  const int row = m + J * 16;
  if constexpr (MODE >= 3) {
    store_gated<MODE - 3, INSIDE>((bf16*)Cbase, row, nb / 2 + P * 16 + g * 4, M, N / 2, ldc, a, b);
  } else {
    store_fragment<MODE, INSIDE>(C, row, nb + (2 * P) * 16 + g * 4, M, N, ldc, a, vec_store);
    store_fragment<MODE, INSIDE>(C, row, nb + (2 * P + 1) * 16 + g * 4, M, N, ldc, b, vec_store);
  }
}

template <int MODE, bool INSIDE, int... I>
__device__ __forceinline__ void wide_stores(std::integer_sequence<int, I...>, void* C, void* Cbase, int m, int nb, int g, int M, int N,
                                            int ldc, bool vec_store) {
  (wide_store<MODE, INSIDE, I / 8, I % 8>(C, Cbase, m, nb, g, M, N, ldc, vec_store), ...);
}

// The same through LDS, for bfloat16 outputs of tiles whose columns lie inside the matrix, with 16-byte
// aligned rows (`rows` of the wave tile's 128 exist): a lane's four values of a row go into the wave's own part of LDS (rows padded by 16
// bytes: conflict-free), then every lane takes 16 bytes of a row back, so that a store instruction
// writes whole 128-byte lines (four rows' worth) instead of 32-byte pieces of sixteen rows. The pieces
// cost four times the requests at the L2, and a tile's stores then took as long as ten slabs of products.
constexpr int WIDE_STAGED_BYTES = 128 * (256 + 16);  // per wave: 128 rows of 128 bf16
template <int MODE, int P, int J>
__device__ __forceinline__ void wide_stage(unsigned char* part, int r, int g) {
  const floatx4 a = wide_acc<(2 * P) * 8 + J>(), b = wide_acc<(2 * P + 1) * 8 + J>();
  constexpr int STRIDE = (MODE >= 3 ? 128 : 256) + 16;
  unsigned char* row = part + (J * 16 + r) * STRIDE;
  union { uint2 u; bf16 e[4]; } o;
  if constexpr (MODE >= 3) {
#pragma unroll
    for (int e = 0; e < 4; ++e) o.e[e] = static_cast<bf16>(activate_fast(a[e], MODE - 3) * b[e]);
    *reinterpret_cast<uint2*>(row + (P * 16 + g * 4) * 2) = o.u;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) o.e[e] = static_cast<bf16>(a[e]);
    *reinterpret_cast<uint2*>(row + ((2 * P) * 16 + g * 4) * 2) = o.u;
#pragma unroll
    for (int e = 0; e < 4; ++e) o.e[e] = static_cast<bf16>(b[e]);
    *reinterpret_cast<uint2*>(row + ((2 * P + 1) * 16 + g * 4) * 2) = o.u;
  }
}
template <int MODE, int... I>
__device__ __forceinline__ void wide_stage_all(std::integer_sequence<int, I...>, unsigned char* part, int r, int g) {
  (wide_stage<MODE, I / 8, I % 8>(part, r, g), ...);
}
// out: the wave tile's first output element; MODE 0 or 3 + an MS_ACT_* number.
template <int MODE>
__device__ __forceinline__ void wide_store_staged(bf16* __restrict__ out, int ldc, int rows, unsigned char* part, int lane) {
  wide_stage_all<MODE>(std::make_integer_sequence<int, 32>{}, part, lane % 16, lane / 16);
  constexpr int CHUNKS = MODE >= 3 ? 8 : 16, STRIDE = CHUNKS * 16 + 16, ROWS = 64 / CHUNKS;
  const int lrow = lane / CHUNKS, ch = lane % CHUNKS;
#pragma unroll 8
  for (int it = 0; it < 128 / ROWS; ++it) {
    const int row = it * ROWS + lrow;
    const uint4 v = *reinterpret_cast<const uint4*>(part + row * STRIDE + ch * 16);
    if (row < rows) *reinterpret_cast<uint4*>(out + (size_t)row * ldc + ch * 8) = v;
  }
}

// The mode is told apart once, not per fragment: each mode's stores are one straight run of code.
template <bool INSIDE>
__device__ __forceinline__ void wide_epilogue(void* C, void* Cbase, int mode, int m, int nb, int g, int M, int N, int ldc, bool vec_store) {
  constexpr auto all = std::make_integer_sequence<int, 32>{};
  static_assert(MS_ACT_COUNT == 2, "one case per activation below");
  switch (mode) {
    case 0: wide_stores<0, INSIDE>(all, C, Cbase, m, nb, g, M, N, ldc, vec_store); break;
    case 1: wide_stores<1, INSIDE>(all, C, Cbase, m, nb, g, M, N, ldc, vec_store); break;
    case 2: wide_stores<2, INSIDE>(all, C, Cbase, m, nb, g, M, N, ldc, vec_store); break;
    case 3: wide_stores<3, INSIDE>(all, C, Cbase, m, nb, g, M, N, ldc, vec_store); break;
    default: wide_stores<4, INSIDE>(all, C, Cbase, m, nb, g, M, N, ldc, vec_store); break;
  }
}

// Names of registers 96 to 255 (VGPRs) and 0 to 255 (AGPRs) for the loop's clobber list.
#define MS_R10(p, t) p #t "0", p #t "1", p #t "2", p #t "3", p #t "4", p #t "5", p #t "6", p #t "7", p #t "8", p #t "9"
#define MS_R100_249(p)                                                                                                  \
  MS_R10(p, 10), MS_R10(p, 11), MS_R10(p, 12), MS_R10(p, 13), MS_R10(p, 14), MS_R10(p, 15), MS_R10(p, 16), MS_R10(p, 17), \
      MS_R10(p, 18), MS_R10(p, 19), MS_R10(p, 20), MS_R10(p, 21), MS_R10(p, 22), MS_R10(p, 23), MS_R10(p, 24)
#define MS_R250_255(p) p "250", p "251", p "252", p "253", p "254", p "255"
#define MS_WIDE_VGPRS "v96", "v97", "v98", "v99", MS_R100_249("v"), MS_R250_255("v")
#define MS_WIDE_AGPRS                                                                                                   \
  MS_R10("a", ), MS_R10("a", 1), MS_R10("a", 2), MS_R10("a", 3), MS_R10("a", 4), MS_R10("a", 5), MS_R10("a", 6),        \
      MS_R10("a", 7), MS_R10("a", 8), MS_R10("a", 9), MS_R100_249("a"), MS_R250_255("a")
__global__ __launch_bounds__(256, 1) void gemm_bf16_wide_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                                void* __restrict__ Cbase, int mode, int M, int N, int Kfull,
                                                                int ldx, int ldc, int k_per, size_t c_split_stride,
                                                                int xcd_rows, int band_cols, int items) {
  constexpr int BM = 256, BN = 256, KS = 64, ROW_BYTES = KS * 2, STAGE_BYTES = (BM + BN) * ROW_BYTES;
  static_assert(STAGE_BYTES == 0x10000, "the loop flips stages by 64 KB");
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];  // 2 * STAGE_BYTES, and 4 * WIDE_STAGED_BYTES for the stores

  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int wm = (wave / 2) * 128, wn = (wave % 2) * 128;
  // A block works through items blockIdx.x, + gridDim.x, ...: one block per CU stays for the whole product, so
  // that a tile's stores drain and the next tile's first loads fly while no block has to end and another
  // to start in between. (The grid is a multiple of 8 or a single round: item L runs on XCD L % 8.)
  for (int item = blockIdx.x; item < items; item += gridDim.x) {
  const TileId id = tile_of_block(item, items, (M + BM - 1) / BM, (N + BN - 1) / BN, xcd_rows, band_cols);
  const int m0 = id.m * BM, n0 = id.n * BN;
  const int k_lo = id.split * k_per;
  const int K = min(Kfull, k_lo + k_per);
  const int slabs = (K - k_lo) / KS;
  void* C = mode == 1 ? (void*)((float*)Cbase + id.split * c_split_stride) : Cbase;

  // Load side: instruction j of this wave fills tile rows (8 wave + j) * 8 .. + 7, a lane 16 bytes of one.
  const int lrow = lane / 8, lslot = lane % 8;
  unsigned xo[8], wo[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int R = (wave * 8 + j) * 8 + lrow;
    const unsigned chunk = (unsigned)((lslot ^ ((R >> 1) & 7)) * 16);
    xo[j] = (unsigned)(min(m0 + R, M - 1) - m0) * (unsigned)ldx * 2u + chunk;
    wo[j] = (unsigned)(min(n0 + R, N - 1) - n0) * (unsigned)Kfull * 2u + chunk;
  }
  const unsigned long long xb = (unsigned long long)(X + (size_t)m0 * ldx + k_lo);
  const unsigned long long wb = (unsigned long long)(W + (size_t)n0 * Kfull + k_lo);
  // The same for every lane, which the compiler cannot tell: into scalar registers by hand.
  const unsigned xb_lo = __builtin_amdgcn_readfirstlane((unsigned)xb), xb_hi = __builtin_amdgcn_readfirstlane((unsigned)(xb >> 32));
  const unsigned wb_lo = __builtin_amdgcn_readfirstlane((unsigned)wb), wb_hi = __builtin_amdgcn_readfirstlane((unsigned)(wb >> 32));
  const unsigned slabs_left = __builtin_amdgcn_readfirstlane((unsigned)slabs);
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
  const unsigned dma = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)wave * 8192u);
  // Read side: the rows of a fragment are base + r with base a multiple of 16, so the slot of chunk c
  // is c ^ (r >> 1) for every fragment; step t reads chunk column 4 t + g.
  const unsigned fr = (unsigned)lane % 16u, fg = (unsigned)lane / 16u, sw = (fr >> 1) & 7u;
  const unsigned raw0 = lds0 + BM * ROW_BYTES + ((unsigned)wn + fr) * ROW_BYTES + ((fg ^ sw) * 16u);
  const unsigned raw1 = lds0 + BM * ROW_BYTES + ((unsigned)wn + fr) * ROW_BYTES + (((4u + fg) ^ sw) * 16u);
  const unsigned rax0 = lds0 + ((unsigned)wm + fr) * ROW_BYTES + ((fg ^ sw) * 16u);
  const unsigned rax1 = lds0 + ((unsigned)wm + fr) * ROW_BYTES + (((4u + fg) ^ sw) * 16u);

// Between the 64 products of a step: a fragment read after every third (all 16 are out 18 products
// before the step ends, so the next step starts without waiting for them; every second or fourth
// measured the same), a load into LDS around every fourth. The loads are best spread as thin as a step
// allows: every third measured 3 % slower, every second in either half of the step 7 %, all 16 right after
// the barrier 11 to 12 %: their LDS writes then crowd out the fragment reads.
#define MS_WIDE_READ_EVERY 3  // a fragment read after products 1, 4, 7, ... of a step
#define MS_WIDE_READ_FIRST 1
#define MS_WIDE_LOAD_EVERY 4  // a load into LDS around products 3, 7, 11, ... of a slab's second step
#define MS_WIDE_LOAD_FIRST 3
#define MS_STR2(x) #x
#define MS_STR(x) MS_STR2(x)
  asm volatile(".set ms_read_every, " MS_STR(MS_WIDE_READ_EVERY) "\n.set ms_read_first, " MS_STR(MS_WIDE_READ_FIRST) "\n.set ms_load_every, " MS_STR(MS_WIDE_LOAD_EVERY) "\n.set ms_load_first, " MS_STR(MS_WIDE_LOAD_FIRST) "\n" R"(
    .macro MS_WIDE_MFMA mi, cw, cx
      v_mfma_f32_16x16x32_bf16 a[(\mi)*4:(\mi)*4+3], v[\cw+((\mi)>>3)*4:\cw+((\mi)>>3)*4+3], v[\cx+((\mi)&7)*4:\cx+((\mi)&7)*4+3], a[(\mi)*4:(\mi)*4+3]
    .endm
    .macro MS_WIDE_READ q, nw, nx, aw, ax
      .if (\q) < 8
        ds_read_b128 v[\nw+(\q)*4:\nw+(\q)*4+3], v[\aw] offset:(\q)*2048
      .else
        ds_read_b128 v[\nx+((\q)-8)*4:\nx+((\q)-8)*4+3], v[\ax] offset:((\q)-8)*2048
      .endif
    .endm
    .macro MS_WIDE_LOAD_TO q
      s_add_u32 m0, s84, (\q)*1024+((\q)>>3)*24576
    .endm
    .macro MS_WIDE_LOAD q
      .if (\q) < 8
        global_load_lds_dwordx4 v[96+(\q)], s[80:81]
      .else
        global_load_lds_dwordx4 v[96+(\q)], s[82:83]
      .endif
    .endm
    .macro MS_WIDE_SLAB_LOADS
      .set ms_q, 0
      .rept 16
        MS_WIDE_LOAD_TO ms_q
        s_nop 0
        MS_WIDE_LOAD ms_q
        .set ms_q, ms_q+1
      .endr
      s_add_u32 s80, s80, 128
      s_addc_u32 s81, s81, 0
      s_add_u32 s82, s82, 128
      s_addc_u32 s83, s83, 0
    .endm
    .macro MS_WIDE_STEP cw, cx, nw, nx, aw, ax, loads
      .set ms_mi, 0
      .rept 64
        .set ms_rq, (ms_mi-ms_read_first)/ms_read_every
        .set ms_lq, (ms_mi-ms_load_first)/ms_load_every
        .if \loads && (ms_mi >= ms_load_first) && ((ms_mi-ms_load_first) == ms_lq*ms_load_every) && (ms_lq < 16)
          MS_WIDE_LOAD_TO ms_lq
        .endif
        MS_WIDE_MFMA ms_mi, \cw, \cx
        .if (ms_mi >= ms_read_first) && ((ms_mi-ms_read_first) == ms_rq*ms_read_every) && (ms_rq < 16)
          MS_WIDE_READ ms_rq, \nw, \nx, \aw, \ax
        .endif
        .if \loads && (ms_mi >= ms_load_first) && ((ms_mi-ms_load_first) == ms_lq*ms_load_every) && (ms_lq < 16)
          MS_WIDE_LOAD ms_lq
        .endif
        .set ms_mi, ms_mi+1
      .endr
    .endm

    v_mov_b32 v96, %[xo0]
    v_mov_b32 v97, %[xo1]
    v_mov_b32 v98, %[xo2]
    v_mov_b32 v99, %[xo3]
    v_mov_b32 v100, %[xo4]
    v_mov_b32 v101, %[xo5]
    v_mov_b32 v102, %[xo6]
    v_mov_b32 v103, %[xo7]
    v_mov_b32 v104, %[wo0]
    v_mov_b32 v105, %[wo1]
    v_mov_b32 v106, %[wo2]
    v_mov_b32 v107, %[wo3]
    v_mov_b32 v108, %[wo4]
    v_mov_b32 v109, %[wo5]
    v_mov_b32 v110, %[wo6]
    v_mov_b32 v111, %[wo7]
    v_mov_b32 v112, %[raw0]
    v_mov_b32 v113, %[raw1]
    v_mov_b32 v114, %[rax0]
    v_mov_b32 v115, %[rax1]
    s_mov_b32 s80, %[xb_lo]
    s_mov_b32 s81, %[xb_hi]
    s_mov_b32 s82, %[wb_lo]
    s_mov_b32 s83, %[wb_hi]
    s_mov_b32 s84, %[dma]
    s_mov_b32 s85, 0x10000
    s_mov_b32 s86, %[slabs]
    s_nop 4
    MS_WIDE_SLAB_LOADS
    s_add_u32 s84, s84, s85
    s_nop 4
    MS_WIDE_SLAB_LOADS
    s_sub_u32 s84, s84, s85
    .set ms_q, 0
    .rept 256
      v_accvgpr_write_b32 a[ms_q], 0
      .set ms_q, ms_q+1
    .endr
    s_waitcnt vmcnt(16)
    s_barrier
    .set ms_q, 0
    .rept 16
      MS_WIDE_READ ms_q, 128, 160, 112, 114
      .set ms_q, ms_q+1
    .endr
  L_ms_wide_loop_%=:
    s_waitcnt lgkmcnt(0)
    MS_WIDE_STEP 128, 160, 192, 224, 113, 115, 0
    v_add_u32 v112, s85, v112
    v_add_u32 v113, s85, v113
    v_add_u32 v114, s85, v114
    v_add_u32 v115, s85, v115
    s_waitcnt vmcnt(0) lgkmcnt(0)
    s_barrier
    s_cmp_gt_u32 s86, 2
    s_cbranch_scc0 L_ms_wide_last_%=
    MS_WIDE_STEP 192, 224, 128, 160, 112, 114, 1
    s_add_u32 s80, s80, 128
    s_addc_u32 s81, s81, 0
    s_add_u32 s82, s82, 128
    s_addc_u32 s83, s83, 0
    s_branch L_ms_wide_join_%=
  L_ms_wide_last_%=:
    MS_WIDE_STEP 192, 224, 128, 160, 112, 114, 0
  L_ms_wide_join_%=:
    s_add_u32 s84, s84, s85
    s_sub_u32 s85, 0, s85
    s_sub_u32 s86, s86, 1
    s_cmp_lg_u32 s86, 0
    s_cbranch_scc1 L_ms_wide_loop_%=
    s_waitcnt vmcnt(0) lgkmcnt(0)
    s_nop 7
    s_nop 7
    s_nop 7
    .purgem MS_WIDE_MFMA
    .purgem MS_WIDE_READ
    .purgem MS_WIDE_LOAD_TO
    .purgem MS_WIDE_LOAD
    .purgem MS_WIDE_SLAB_LOADS
    .purgem MS_WIDE_STEP
  )"
               :
               : [xo0] "v"(xo[0]), [xo1] "v"(xo[1]), [xo2] "v"(xo[2]), [xo3] "v"(xo[3]), [xo4] "v"(xo[4]), [xo5] "v"(xo[5]),
                 [xo6] "v"(xo[6]), [xo7] "v"(xo[7]), [wo0] "v"(wo[0]), [wo1] "v"(wo[1]), [wo2] "v"(wo[2]), [wo3] "v"(wo[3]),
                 [wo4] "v"(wo[4]), [wo5] "v"(wo[5]), [wo6] "v"(wo[6]), [wo7] "v"(wo[7]), [raw0] "v"(raw0), [raw1] "v"(raw1),
                 [rax0] "v"(rax0), [rax1] "v"(rax1), [xb_lo] "s"(xb_lo), [xb_hi] "s"(xb_hi), [wb_lo] "s"(wb_lo),
                 [wb_hi] "s"(wb_hi), [dma] "s"(dma), [slabs] "s"(slabs_left)
               : "memory", "scc", "s80", "s81", "s82", "s83", "s84", "s85", "s86", MS_WIDE_VGPRS, MS_WIDE_AGPRS);

  // The stores' address arithmetic starts from a lane number the compiler cannot see through: what
  // it could work out once for all items it would keep in registers across the loop, of which it has 96
  // there, and spill.
  int lane_now = lane;
  asm volatile("" : "+v"(lane_now));
  const int r = lane_now % 16, g = lane_now / 16;
  const bool vec_store = (ldc % 4 == 0);
  // (gated: the output has N / 2 columns, and a lane's four of them are 8-byte aligned when ldc is a multiple of 4)
  const bool inside = n0 + BN <= N && vec_store;  // the columns; rows are tested where they are stored
  if (inside && (mode == 0 || mode >= 3) && ldc % 8 == 0 && (size_t)Cbase % 16 == 0) {
    unsigned char* part = lds + wave * WIDE_STAGED_BYTES;
    const int rows = M - (m0 + wm);  // of the wave tile's 128 that exist
    static_assert(MS_ACT_COUNT == 2, "one case per activation below");
    if (mode == 0) wide_store_staged<0>((bf16*)Cbase + (size_t)(m0 + wm) * ldc + n0 + wn, ldc, rows, part, lane_now);
    else if (mode == 3) wide_store_staged<3>((bf16*)Cbase + (size_t)(m0 + wm) * ldc + (n0 + wn) / 2, ldc, rows, part, lane_now);
    else wide_store_staged<4>((bf16*)Cbase + (size_t)(m0 + wm) * ldc + (n0 + wn) / 2, ldc, rows, part, lane_now);
    __syncthreads();  // the next item's loads go where other waves may still be reading their parts
  } else if (inside) {
    wide_epilogue<true>(C, Cbase, mode, m0 + wm + r, n0 + wn, g, M, N, ldc, vec_store);
  } else {
    wide_epilogue<false>(C, Cbase, mode, m0 + wm + r, n0 + wn, g, M, N, ldc, vec_store);
  }
  }
}

// ---------------------------------------------------------------------------------------------
// Small-M kernel: M <= 16 * MB rows of X (a decode step). Pure weight streaming: a wave owns 16 weight
// rows and a slice of K; per step of 64 k each lane loads 32 bytes of its weight row and issues two
// MFMAs per 16-row block of X. Without SHARED (MB == 1 only) the matching 32 bytes of an X row come
// straight from global memory (no LDS, no barrier: the cheapest form where launch and latency decide);
// with SHARED the block's four waves stage the X slab of their common K slice in LDS, so that X passes
// through the caches once per 64 weight rows instead of once per 16 (it is half the weights' bytes at
// 8 rows, and what then limits large matrices). K is split over the grid so
// that even a 1024-row matrix gives every CU several waves; each split writes float partial sums
// P[split, M, N], which the caller's next kernel (or the reduction below) sums in ascending split
// order. The number of splits depends on N, K and on the class of M (up to 4, 5 to 16, above 16), not on
// M itself: within a class a row's result does not depend on the batch it is in.
#define SMALL_SLAB 256  // k per iteration: four steps of 64
#define XS_STRIDE (SMALL_SLAB + 8)
// Up to 16 rows: the shared X slab is used from this many rows and this many weights on (measured:
// 8 to 20 % faster at 8 to 16 rows and 8B / 32B layer shapes, slower below 4 M weights).
constexpr int SMALL_SHARED_MIN_ROWS = 4;
constexpr long SMALL_SHARED_MIN_WEIGHTS = 16L << 20;

template <int MB, bool SHARED>
__global__ __launch_bounds__(256) void gemm_bf16_small_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                              float* __restrict__ P, int M, int N, int K, int ldx,
                                                              int steps_per_split, int splits) {
  __shared__ __attribute__((aligned(16))) bf16 xs[SHARED ? MB * 16 * XS_STRIDE : 8];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  // The split index runs fastest over the grid: blocks that are resident together read neighbouring
  // k ranges of the same weight rows, which together are whole rows, instead of the same k range of
  // rows that lie a power of two apart (those would queue up on a few memory channels).
  const int split = blockIdx.x % splits, row_block = blockIdx.x / splits;
  const int nb = (row_block * (blockDim.x / WAVE) + wave) * 16;  // without a shared slab: one wave per block
  const int n = nb + r;
  const int k_begin = split * steps_per_split * 64;
  const int k_end = min(K, k_begin + steps_per_split * 64);
  const bool vecx = (K % 8 == 0) && (ldx % 8 == 0), vecw = (K % 8 == 0);
  const bool rows_in = vecw && nb + 16 <= N;  // the same for the whole wave

  floatx4 acc[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int k0 = k_begin; k0 < k_end; k0 += SMALL_SLAB) {
    // This lane's weights of the slab: per step of 64 k, 16 consecutive k at offset 16 g. Chunks at or
    // beyond k_end are asked for at K, where load_chunk yields zeros. A slab that lies wholly inside
    // the matrix is loaded without any test, so that all its loads go out back to back.
    const bool whole = k0 + SMALL_SLAB <= k_end;
    // Shared slab: this thread's share of the X slab goes out first (it comes from the cache and is back
    // while the weights are still on their way), so that staging it in LDS costs no waiting of its own.
    constexpr int XPT = SHARED ? MB * 16 * (SMALL_SLAB / 8) / 256 : 1;  // 16-byte chunks per thread
    Chunk xr[XPT];
    if (SHARED) {
      if (vecx && whole) {
        const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < XPT; ++j) {
          const int c = tid + j * 256, m = c / (SMALL_SLAB / 8), kc = (c % (SMALL_SLAB / 8)) * 8;
          const uint4 v = *reinterpret_cast<const uint4*>(X + (size_t)min(m, M - 1) * ldx + k0 + kc);
          xr[j].u = m < M ? v : zero;
        }
      } else {
#pragma unroll
        for (int j = 0; j < XPT; ++j) {
          const int c = tid + j * 256, m = c / (SMALL_SLAB / 8), kc = (c % (SMALL_SLAB / 8)) * 8;
          const int k = k0 + kc;
          xr[j] = load_chunk(X, m, M, k < k_end ? k : K, K, ldx, vecx);
        }
      }
    }
    Chunk w[SMALL_SLAB / 64][2];
    if (rows_in && whole) {
      const bf16* wp = W + (size_t)n * K + k0 + g * 16;
#pragma unroll
      for (int u = 0; u < SMALL_SLAB / 64; ++u) {
        w[u][0].u = *reinterpret_cast<const uint4*>(wp + u * 64);
        w[u][1].u = *reinterpret_cast<const uint4*>(wp + u * 64 + 8);
      }
    } else {
#pragma unroll
      for (int u = 0; u < SMALL_SLAB / 64; ++u) {
        const int k = k0 + u * 64 + g * 16;
        const int kw = k < k_end ? k : K;
        w[u][0] = load_chunk(W, n, N, kw, K, K, vecw);
        w[u][1] = load_chunk(W, n, N, kw + 8, K, K, vecw);
      }
    }
    if (!SHARED) {
      static_assert(SHARED || MB == 1, "more than 16 rows need the shared slab");
      Chunk x[SMALL_SLAB / 64][2];
      if (vecx && whole) {
        const bf16* xp = X + (size_t)min(r, M - 1) * ldx + k0 + g * 16;  // rows beyond M: read row M - 1, use zeros
        const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int u = 0; u < SMALL_SLAB / 64; ++u) {
          const uint4 a = *reinterpret_cast<const uint4*>(xp + u * 64);
          const uint4 b = *reinterpret_cast<const uint4*>(xp + u * 64 + 8);
          x[u][0].u = r < M ? a : zero;
          x[u][1].u = r < M ? b : zero;
        }
      } else {
#pragma unroll
        for (int u = 0; u < SMALL_SLAB / 64; ++u) {
          const int k = k0 + u * 64 + g * 16;
          const int kw = k < k_end ? k : K;
          x[u][0] = load_chunk(X, r, M, kw, K, ldx, vecx);
          x[u][1] = load_chunk(X, r, M, kw + 8, K, ldx, vecx);
        }
      }
#pragma unroll
      for (int u = 0; u < SMALL_SLAB / 64; ++u) {
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][0].v, x[u][0].v, acc[0], 0, 0, 0);
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][1].v, x[u][1].v, acc[0], 0, 0, 0);
      }
    } else {
      __syncthreads();  // the previous slab has been consumed
#pragma unroll
      for (int j = 0; j < XPT; ++j) {
        const int c = tid + j * 256, m = c / (SMALL_SLAB / 8), kc = (c % (SMALL_SLAB / 8)) * 8;
        *reinterpret_cast<uint4*>(&xs[m * XS_STRIDE + kc]) = xr[j].u;
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < SMALL_SLAB / 64; ++u) {
#pragma unroll
        for (int i = 0; i < MB; ++i) {
          const bf16* xp = &xs[(i * 16 + r) * XS_STRIDE + u * 64 + g * 16];
          const bf16x8 x0 = *reinterpret_cast<const bf16x8*>(xp);
          const bf16x8 x1 = *reinterpret_cast<const bf16x8*>(xp + 8);
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][0].v, x0, acc[i], 0, 0, 0);
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][1].v, x1, acc[i], 0, 0, 0);
        }
      }
    }
  }
  // acc[i][e] = C[m = 16 i + r][n = nb + 4 g + e]
  float* dst = P + (size_t)split * M * N;
  if (SHARED && MB == 1 && N % 4 == 0) {
    // A wave's own store would put 64 bytes into each of up to 16 rows: half cache lines, which the
    // memory system takes at a fraction of its rate (at 8 rows the partial sums of a 24576 x 4096
    // matrix cost as much as 15 % of its weights). The block's four waves meet in LDS instead and
    // write their 64 columns of a row as one run of 256 bytes.
    float* outs = reinterpret_cast<float*>(xs);  // 16 rows x 64 columns
    static_assert(!SHARED || MB * 16 * XS_STRIDE * 2 >= 16 * 64 * 4, "the X slab's memory holds the block's results");
    __syncthreads();  // every wave is done with the last slab
    *reinterpret_cast<floatx4*>(&outs[r * 64 + wave * 16 + g * 4]) = acc[0];
    __syncthreads();
    const int m = tid / 16, n = row_block * 64 + (tid % 16) * 4;
    if (m < M && n < N) *reinterpret_cast<floatx4*>(dst + (size_t)m * N + n) = *reinterpret_cast<const floatx4*>(&outs[m * 64 + (tid % 16) * 4]);
    return;
  }
#pragma unroll
  for (int i = 0; i < MB; ++i) store4(dst, 1, i * 16 + r, nb + g * 4, M, N, N, acc[i], N % 4 == 0);
}

// C (mode 0 bf16 / 1 float / 2 float +=) from the partial sums, in ascending split order.
__global__ void splitk_reduce_kernel(const float* __restrict__ P, void* __restrict__ C, int mode, int splits, int M,
                                     int N, int ldc) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x, m = blockIdx.y;
  if (n >= N) return;
  const float v = sum_splits(P + (size_t)m * N + n, splits, (size_t)M * N);
  const size_t at = (size_t)m * ldc + n;
  if (mode == 0) ((bf16*)C)[at] = static_cast<bf16>(v);
  else if (mode == 1) ((float*)C)[at] = v;
  else ((float*)C)[at] += v;
}

extern "C" int ms_splitk_reduce(const float* P, void* C, int mode, int splits, int M, int N, int ldc, hipStream_t st) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (splits < 1 || ldc < N || mode < 0 || mode > 2 || M > 65535) return MS_BAD_ARG;
  splitk_reduce_kernel<<<dim3((N + 255) / 256, M), 256, 0, st>>>(P, C, mode, splits, M, N, ldc);
  return launch_status();
}

// Weight memory that one band of tile columns may span: well inside the 256 MB last-level cache. Without
// bands the 32B gate/up product (524 MB of weights, re-read by each of 16 row tiles) ran at 650 TFLOP/s,
// bound by memory; with them at 850-950.
constexpr long DMA_BAND_BYTES = 96L << 20;

// How the blocks of a grid of BM x BN tiles walk it (the two last arguments of the kernels).
struct TileWalk {
  int xcd_rows, band_cols;
};
static TileWalk tile_walk(int M, int N, int K, int BM, int BN) {
  // How the XCDs share the tiles: as a grid of xcd_rows x 8 / xcd_rows rectangles where the tile counts
  // divide, chosen so that the bytes all XCDs read together (its share of the activations once per
  // XCD column, its share of the weights once per XCD row) are fewest, if that is under 0.6 of what
  // columns in turn (0) read: measured, a smaller advantage does not pay (N = 1024 at 2,048 rows: 10 %
  // faster; N = 4096 to 6144: 2 to 5 % slower).
  const int row_tiles = (M + BM - 1) / BM, col_tiles = (N + BN - 1) / BN;
  int xcd_rows = 0;
  long least = (8L * M + N) * 6 / 10;
  for (int pm = 2; pm <= 8; pm *= 2) {
    const int pn = 8 / pm;
    if (row_tiles % pm || col_tiles % pn) continue;
    const long cost = (long)pn * M + (long)pm * N;
    if (cost < least) {
      least = cost;
      xcd_rows = pm;
    }
  }
  // Weight tile columns of a band: what fits in DMA_BAND_BYTES but at least 32 over all XCDs (four per
  // XCD: with fewer, many blocks of an XCD wait for the same slab at the same time, which measured
  // slower than no bands), then evened out over the bands; a multiple of eight where the XCDs take
  // columns in turn.
  long band_cols = DMA_BAND_BYTES / ((long)BN * K * 2);
  if (band_cols < 32) band_cols = 32;
  if (xcd_rows == 0) {
    const long bands = (col_tiles + band_cols - 1) / band_cols;
    band_cols = ((col_tiles + bands - 1) / bands + 7) / 8 * 8;
  } else {
    const int sub_cols = col_tiles / (8 / xcd_rows);
    band_cols = band_cols / (8 / xcd_rows);
    const long bands = (sub_cols + band_cols - 1) / band_cols;
    band_cols = (sub_cols + bands - 1) / bands;
  }
  return TileWalk{xcd_rows, (int)band_cols};
}

template <int BM, int BN, int KS, int STAGES, int BLOCKS_PER_CU, int WR = 2, int WC = 2>
static int launch_dma(const bf16* x, const bf16* w, void* C, int mode, int M, int N, int K, int ldx, int ldc, int k_per,
                      size_t stride, int splits, hipStream_t st) {
  constexpr int lds_bytes = STAGES * (BM + BN) * KS * 2;
  static bool ready = false;  // more than 64 KB of LDS has to be asked for once per kernel
  if (!ready) {
    if (hipFuncSetAttribute((const void*)gemm_bf16_dma_kernel<BM, BN, KS, STAGES, BLOCKS_PER_CU, WR, WC>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
      return MS_LAUNCH_FAILED;
    ready = true;
  }
  const long blocks = (long)((N + BN - 1) / BN) * ((M + BM - 1) / BM) * splits;
  if (blocks > 0x7fffffffL) return MS_BAD_ARG;
  const TileWalk walk = tile_walk(M, N, K, BM, BN);
  gemm_bf16_dma_kernel<BM, BN, KS, STAGES, BLOCKS_PER_CU, WR, WC><<<(unsigned)blocks, WR * WC * WAVE, lds_bytes, st>>>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, walk.xcd_rows, walk.band_cols);
  return launch_status();
}

// The wide tile's loop adds 32-bit byte offsets of up to 255 rows to a tile's base.
static bool wide_tile_offsets_fit(int ldx, int K) { return ldx < (1 << 22) && K < (1 << 22); }

// Compute units of the current device (asked once per device).
static int compute_units() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    cached[dev] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n >= 8) ? n : 256;
  }
  return cached[dev];
}

// The 256 x 256 tile: four waves with the loop written out where every split has at least two slabs and a
// tile's rows lie within 4 GB of its first (the loop adds 32-bit offsets to a tile's base), else 128 x 128 tiles.
static int launch_256(const bf16* x, const bf16* w, void* C, int mode, int M, int N, int K, int ldx, int ldc, int k_per,
                      size_t stride, int splits, hipStream_t st) {
  const int last_slabs = (K - (splits - 1) * k_per) / BK;  // of the last split, the shortest
  if (last_slabs < 2 || k_per < 2 * BK || !wide_tile_offsets_fit(ldx, K))
    return launch_dma<128, 128, BK, 2, 2>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
  constexpr int lds_bytes = 4 * WIDE_STAGED_BYTES;  // the loop's two stages are 128 KB of it
  static_assert(lds_bytes >= 2 * (256 + 256) * BK * 2 && lds_bytes <= 160 * 1024, "LDS of the wide tile");
  static bool ready = false;
  if (!ready) {
    if (hipFuncSetAttribute((const void*)gemm_bf16_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
      return MS_LAUNCH_FAILED;
    ready = true;
  }
  const long items = (long)((N + 255) / 256) * ((M + 255) / 256) * splits;
  if (items > 0x7fffffffL) return MS_BAD_ARG;
  const TileWalk walk = tile_walk(M, N, K, 256, 256);
  const int cus = compute_units();
  const int blocks = items <= cus ? (int)items : cus / 8 * 8;
  gemm_bf16_wide_kernel<<<(unsigned)blocks, 256, lds_bytes, st>>>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, walk.xcd_rows, walk.band_cols, (int)items);
  return launch_status();
}

// Tile shape of a product with at least 256 tiles of 128 x 128: 128-row tiles of four waves, 64 to 192
// columns wide, two blocks per CU (512 run at once), or 256 x 256 tiles of four waves with wave tiles of
// 128 x 128 (one block per CU that stays and takes tiles in turn; a wave reads 16 fragments for 64
// products where the 64 x 64 wave tile reads 8 for 16). The choice is the least predicted time. For
// the 128-row tiles: a fixed part (launch, first slab, stores) plus, per slab of 64 k, the time of a
// round of blocks; a block that has a CU to itself is faster than one that shares it, so a last round
// of up to 256 blocks counts less than a full one. For the 256 x 256 tile: a fixed part per launch and,
// per round of 256 tiles, another (first slab, stores) plus its slabs, a last round of up to 128 tiles counting less per slab (half
// the chip idles: less traffic). The figures (microseconds) are fits to products of 384 to 8,192 rows,
// 1,024 to 24,576 columns and K of 1,024, 4,096 and 12,288 timed with every shape (270 for the 128-row
// tiles, 177 for the 256 x 256 tile as it is now); over those 177 picking by them takes 0.5 % longer
// in total than the best shape of each, 1.2 % per product on average and 29 % at worst, where rules by
// tile counts alone lost up to 28 % in whole layers (2,048 x 5,120 x 12,288: 160 columns make exactly
// 512 tiles).
struct TileShape {
  int cols;      // 256 stands for the 256 x 256 tile
  float fixed;   // per launch
  float alone;   // per slab, a last round with one block per CU (256: with up to 128 tiles)
  float shared;  // per slab, a round with two blocks per CU (256: any other round)
  float round;   // per round of tiles (256 only)
};
static const TileShape TILE_SHAPES[5] = {
    {128, 7.7f, 0.611f, 0.976f, 0.f}, {64, 6.1f, 0.456f, 0.627f, 0.f}, {160, 8.8f, 0.707f, 1.168f, 0.f},
    {192, 9.1f, 0.803f, 1.364f, 0.f}, {256, 4.5f, 0.997f, 1.306f, 3.9f}};

// Whether the 256 x 256 tile takes a product of this K in this many splits: its loop needs two slabs.
static bool wide_tile_runs(int K, int splits) {
  const int slabs = (K + BK - 1) / BK, per = (slabs + splits - 1) / splits;
  return per >= 2 && slabs - (splits - 1) * per >= 2;
}

// `pairs`: the gated epilogue needs an even number of 16-column fragments per wave, which 160 columns
// over two waves are not.
static int pick_tile_cols(int M, int N, int K, int splits, bool pairs, float* predicted = nullptr) {
  const float slabs = (float)((K + BK - 1) / BK) / splits;
  int best = 128;
  float least = 0.f;
  for (int i = 0; i < 5; ++i) {
    const TileShape& t = TILE_SHAPES[i];
    if (pairs && t.cols == 160) continue;
    float time;
    if (t.cols == 256) {
      const long tiles = (long)((M + 255) / 256) * ((N + 255) / 256) * splits;
      const long rest = tiles % 256;
      if (!wide_tile_runs(K, splits)) continue;
      time = t.fixed + (float)(tiles / 256) * (t.round + slabs * t.shared) +
             (rest == 0 ? 0.f : t.round + slabs * (rest <= 128 ? t.alone : t.shared));
    } else {
      const long tiles = (long)((M + 127) / 128) * ((N + t.cols - 1) / t.cols) * splits;
      const long rest = tiles % 512;
      time = t.fixed + slabs * ((float)(tiles / 512) * t.shared + (rest == 0 ? 0.f : rest <= 256 ? t.alone : t.shared));
    }
    if (i == 0 || time < least) {
      least = time;
      best = t.cols;
    }
  }
  if (predicted) *predicted = least;
  return best;
}

static int launch_picked(int cols, const bf16* x, const bf16* w, void* C, int mode, int M, int N, int K, int ldx, int ldc,
                         int k_per, size_t stride, int splits, hipStream_t st) {
  switch (cols) {
    case 256: return launch_256(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
    case 192: return launch_dma<128, 192, BK, 2, 2>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
    case 160: return launch_dma<128, 160, BK, 2, 2>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
    case 64: return launch_dma<128, 64, BK, 2, 2>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
    default: return launch_dma<128, 128, BK, 2, 2>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
  }
}

// Splits of K for the small-M kernel: one slab (four 64-k steps) per wave, so that a wave issues all
// its loads at once, unless that would make more waves than the chip holds a few times over (then
// slices of several whole slabs). With up to 4 rows the partial sums are small beside the weights
// and 32768 waves are allowed; above that 8192: the partial sums cost more than their bytes (at 8
// rows a 24576 x 4096 matrix writes 12 MB of them in 16 splits, 6 % of its weights, and takes 15 %
// longer than at 1 row; in 4 splits half of that). At most 16 splits: the kernel that sums them up
// reads every one. The count depends on M only through its class (up to 4, 5 to 16, above 16).
#define SMALL_MAX_SPLITS 16
static int small_slabs_per_split(int M, int N, int K) {
  const int slabs = (K + SMALL_SLAB - 1) / SMALL_SLAB;
  const int row_blocks = (N + 15) / 16;
  const int waves = M <= 4 ? 32768 : 8192;
  int s = slabs;
  const int most = waves / row_blocks > 0 ? waves / row_blocks : 1;
  if (s > most) s = most;
  if (s > SMALL_MAX_SPLITS) s = SMALL_MAX_SPLITS;
  return (slabs + s - 1) / s;
}

// 16 < M <= 64 and K a multiple of 64: the product runs as tiles of 64 rows of the kernel whose slabs go
// straight into LDS (it streams the weights faster than the four-wave small-M kernel: 2.9 -> 4.4 TB/s
// at the 8B shapes), with K split so that about 768 blocks are in the grid (384 for matrices of up to
// 16 MB, where the partial sums weigh as much as the weights: measured, 1.7 % of a batch-64 step of the
// 0.6B shape), at most 16 splits and at least two slabs per split. Every block loads its slab of the
// rows beside its slab of the weights, from the L2 but over the same path, so a tile of 64 columns moves
// as many bytes of rows as of weights. Large matrices, which have columns to spare, take wider tiles:
// 128 columns from 224 MB on (three blocks per CU), 256 columns from 400 MB on (two blocks per CU,
// about 384 blocks). Measured at 64 rows with the weights from memory: the 32B gate/up product 132 ->
// 114 us and down 65 -> 57, a decode step of the 32B shape at batch 64 8.5 % faster; smaller matrices
// lose with wider tiles (fewer blocks, or more splits and partial sums), and the 8B gate/up product
// (201 MB), 7 us faster on its own with 128 columns, made the model's step no faster.
static bool small_runs_as_tiles(int M, int K) { return M > 16 && K % BK == 0; }

static int small_tile_cols(int N, int K) {
  const long bytes = (long)N * K * 2;
  return bytes >= (400L << 20) ? 256 : bytes >= (224L << 20) ? 128 : 64;
}

static int tile_slabs_per_split(int N, int K) {
  const int slabs = K / BK;
  const int width = small_tile_cols(N, K);
  const int cols = (N + width - 1) / width;
  const int target = (long)N * K * 2 <= (16L << 20) || width == 256 ? 384 : 768;
  int s = (target + cols - 1) / cols;
  if (s > SMALL_MAX_SPLITS) s = SMALL_MAX_SPLITS;
  if (s > slabs / 2) s = slabs / 2;
  if (s < 1) s = 1;
  return (slabs + s - 1) / s;
}

// Columns of the tiles that a product of 17 to 64 rows (K a multiple of 64) runs as: for tests that
// must know which instance they have reached.
extern "C" int ms_gemm_bf16_small_tile_cols(int N, int K) { return small_tile_cols(N, K); }

extern "C" int ms_gemm_bf16_small_splits(int M, int N, int K) {
  if (small_runs_as_tiles(M, K)) {
    const int per = tile_slabs_per_split(N, K);
    return (K / BK + per - 1) / per;
  }
  const int slabs = (K + SMALL_SLAB - 1) / SMALL_SLAB;
  const int per = small_slabs_per_split(M, N, K);
  return (slabs + per - 1) / per;  // no empty split
}

// X [M <= 64, K] * W [N, K]^T. `partials` holds splits * M * N floats (splits from
// ms_gemm_bf16_small_splits). With reduce != 0 the partial sums are folded into C here; otherwise the
// caller's next kernel sums them.
extern "C" int ms_gemm_bf16_small(const void* X, const void* W, float* partials, void* C, int mode, int reduce, int M,
                                  int N, int K, int ldx, int ldc, hipStream_t st) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (M > 64 || K <= 0 || ldx < K || partials == nullptr) return MS_BAD_ARG;
  const int splits = ms_gemm_bf16_small_splits(M, N, K);
  if (small_runs_as_tiles(M, K) && ldx % 8 == 0) {
    const int k_per = tile_slabs_per_split(N, K) * BK;
    const int width = small_tile_cols(N, K);
    const int rc = width == 256   ? launch_dma<64, 256, BK, 2, 2, 1, 4>((const bf16*)X, (const bf16*)W, partials, 1, M, N, K, ldx, N,
                                                                         k_per, (size_t)M * N, splits, st)
                   : width == 128 ? launch_dma<64, 128, BK, 2, 3, 1, 4>((const bf16*)X, (const bf16*)W, partials, 1, M, N, K, ldx, N,
                                                                         k_per, (size_t)M * N, splits, st)
                                  : launch_dma<64, 64, BK, 2, 4>((const bf16*)X, (const bf16*)W, partials, 1, M, N, K, ldx, N, k_per,
                                                                 (size_t)M * N, splits, st);
    if (rc != MS_OK) return rc;
    if (reduce) {
      if (C == nullptr || ldc < N || mode < 0 || mode > 2) return MS_BAD_ARG;
      splitk_reduce_kernel<<<dim3((N + 255) / 256, M), 256, 0, st>>>(partials, C, mode, splits, M, N, ldc);
    }
    return launch_status();
  }
  if (small_runs_as_tiles(M, K)) return MS_BAD_ARG;  // the split count was made for the tile kernel
  const int per = small_slabs_per_split(M, N, K) * (SMALL_SLAB / 64);
  const long wave_blocks = (long)((N + 15) / 16) * splits, wide_blocks = (long)((N + 63) / 64) * splits;
  if (wave_blocks > 0x7fffffffL) return MS_BAD_ARG;
  const bf16* x = (const bf16*)X;
  const bf16* w = (const bf16*)W;
  // Without a shared X slab the waves of a block have nothing in common: single-wave blocks spread
  // evenly over the CUs. Both forms add up the same products in the same order.
  const bool shared = M >= SMALL_SHARED_MIN_ROWS && (long)N * K >= SMALL_SHARED_MIN_WEIGHTS;
  if (M <= 16 && !shared) gemm_bf16_small_kernel<1, false><<<(unsigned)wave_blocks, WAVE, 0, st>>>(x, w, partials, M, N, K, ldx, per, splits);
  else if (M <= 16) gemm_bf16_small_kernel<1, true><<<(unsigned)wide_blocks, 256, 0, st>>>(x, w, partials, M, N, K, ldx, per, splits);
  else if (M <= 32) gemm_bf16_small_kernel<2, true><<<(unsigned)wide_blocks, 256, 0, st>>>(x, w, partials, M, N, K, ldx, per, splits);
  else gemm_bf16_small_kernel<4, true><<<(unsigned)wide_blocks, 256, 0, st>>>(x, w, partials, M, N, K, ldx, per, splits);
  if (reduce) {
    if (C == nullptr || ldc < N || mode < 0 || mode > 2) return MS_BAD_ARG;
    splitk_reduce_kernel<<<dim3((N + 255) / 256, M), 256, 0, st>>>(partials, C, mode, splits, M, N, ldc);
  }
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Gated feed-forward input for few rows (M <= 16 MB): out[m, i] = act(x . gate_i) * (x . up_i), bf16
// [M, inter], from W [2 inter, K] that holds alternating blocks of 16 gate rows and 16 up rows. One
// block of 8 waves per 16 outputs: waves 0-3 take the gate rows, waves 4-7 the up rows, wave w of each
// four the K slabs w, w + 4, ... (one slab each up to K = 1024: all loads of the block in flight at
// once, 8 KB of weights per wave as in the split product, and the same slab of every 16 rows of X, which
// comes from the cache). The eight partial results meet in LDS; wave i % 8 adds those of rows 16 i ..
// in wave order, applies the activation and stores. No partial sums leave the block and no second
// kernel runs. K must be a multiple of 256 and rows 16-byte aligned.
// (ACT is a template parameter here: the kernel is a chain of latencies, and the choice inside it measured 0.6 % of
// a decode step of one row.)
template <int MB, int ACT>
__global__ __launch_bounds__(512) void gemm_bf16_small_gated_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                                    bf16* __restrict__ out, int M, int inter, int K,
                                                                    int ldx) {
  __shared__ float red[8][MB][WAVE][4];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  const int nb = blockIdx.x * 32 + (wave / 4) * 16;  // first weight row of this wave's block of 16
  floatx4 acc[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16* wp = W + (size_t)(nb + r) * K + g * 16;
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (int k0 = (wave % 4) * SMALL_SLAB; k0 < K; k0 += 4 * SMALL_SLAB) {
    Chunk a[SMALL_SLAB / 64][2], x[MB][SMALL_SLAB / 64][2];
#pragma unroll
    for (int u = 0; u < SMALL_SLAB / 64; ++u) {
      a[u][0].u = *reinterpret_cast<const uint4*>(wp + k0 + u * 64);
      a[u][1].u = *reinterpret_cast<const uint4*>(wp + k0 + u * 64 + 8);
    }
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      const int m = i * 16 + r;
      const bf16* xp = X + (size_t)min(m, M - 1) * ldx + g * 16;  // rows beyond M: read row M - 1, use zeros
#pragma unroll
      for (int u = 0; u < SMALL_SLAB / 64; ++u) {
        const uint4 lo = *reinterpret_cast<const uint4*>(xp + k0 + u * 64);
        const uint4 hi = *reinterpret_cast<const uint4*>(xp + k0 + u * 64 + 8);
        x[i][u][0].u = m < M ? lo : zero;
        x[i][u][1].u = m < M ? hi : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < SMALL_SLAB / 64; ++u)
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][0].v, x[i][u][0].v, acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][1].v, x[i][u][1].v, acc[i], 0, 0, 0);
      }
  }
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][i][lane][e] = acc[i][e];
  __syncthreads();
  // Wave w finishes the rows 16 i + r of every i with i % 8 == w; this lane: outputs 16 blockIdx.x + 4 g + e.
  for (int i = wave; i < MB; i += 8) {
    const int m = i * 16 + r;
    if (m >= M) continue;
    union { uint2 u; bf16 e[4]; } o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float gate = 0.f, up = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        gate += red[w][i][lane][e];
        up += red[4 + w][i][lane][e];
      }
      o.e[e] = static_cast<bf16>(activate(gate, ACT) * up);
    }
    *reinterpret_cast<uint2*>(out + (size_t)m * inter + blockIdx.x * 16 + g * 4) = o.u;
  }
}

// out bf16 [M, inter] = act(X gate^T) * (X up^T) (act: an MS_ACT_* number) for W [2 inter, K] with gate and up rows in
// alternating blocks of 16. MS_UNSUPPORTED for shapes no fused kernel takes (the caller then runs the
// product and the activation separately): K no multiple of 64 (of 256 for M <= 64) or unaligned rows,
// more K than a block of the small kernel should walk alone (2048 up to 16 rows, 1024 up to 32), 33 to
// 64 rows of a large matrix (those stream the weights with K split over blocks).
extern "C" int ms_gemm_bf16_gated(const void* X, const void* W, void* out, int M, int inter, int K, int ldx, int act,
                                  hipStream_t st) {
  if (M <= 0 || inter <= 0) return MS_OK;
  if (K <= 0 || ldx < K || act < 0 || act >= MS_ACT_COUNT) return MS_BAD_ARG;
  const int gated = 3 + act;  // the tile kernel's mode
  if (inter % 16 || ldx % 8) return MS_UNSUPPORTED;
  const bf16* x = (const bf16*)X;
  const bf16* w = (const bf16*)W;
  const int N = 2 * inter;
  if (M <= 16) {
    if (K % SMALL_SLAB || K / SMALL_SLAB > 8) return MS_UNSUPPORTED;
    if (act == MS_ACT_SILU) gemm_bf16_small_gated_kernel<1, MS_ACT_SILU><<<inter / 16, 512, 0, st>>>(x, w, (bf16*)out, M, inter, K, ldx);
    else gemm_bf16_small_gated_kernel<1, MS_ACT_GELU_TANH><<<inter / 16, 512, 0, st>>>(x, w, (bf16*)out, M, inter, K, ldx);
    return launch_status();
  }
  if (M <= 32 && K % SMALL_SLAB == 0 && K / SMALL_SLAB <= 4) {
    // 17 to 32 rows: the same kernel with the block's rows of X from the cache, where one round of
    // slabs covers K (each wave then holds its slab of every row at once): 7.8 against 9.2 us at the
    // 0.6B shape. Larger K streams the weights with K split over blocks and runs the activation as a
    // kernel of its own.
    if (act == MS_ACT_SILU) gemm_bf16_small_gated_kernel<2, MS_ACT_SILU><<<inter / 16, 512, 0, st>>>(x, w, (bf16*)out, M, inter, K, ldx);
    else gemm_bf16_small_gated_kernel<2, MS_ACT_GELU_TANH><<<inter / 16, 512, 0, st>>>(x, w, (bf16*)out, M, inter, K, ldx);
    return launch_status();
  }
  if (K % BK) return MS_UNSUPPORTED;
  if (M <= 64) {
    // 33 to 64 rows (one row of 64 x 64 tiles): the tile kernel with the activation in its epilogue
    // where the matrix is small enough that K need not be split to keep the chip busy.
    if (M > 32 && (long)N * K * 2 <= (16L << 20) && (N + 63) / 64 >= 96)
      return launch_dma<64, 64, BK, 2, 4>(x, w, out, gated, M, N, K, ldx, inter, K, 0, 1, st);
    return MS_UNSUPPORTED;
  }
  const long big = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (big >= 256) return launch_picked(pick_tile_cols(M, N, K, 1, true), x, w, out, gated, M, N, K, ldx, inter, K, 0, 1, st);
  // 64 x 64 tiles from 128 of them on: half the CUs without a split of K still beat the split product
  // followed by the activation kernel (10.2 against 11.8 to 13.1 us at 65 to 128 rows of the 0.6B shape).
  if ((long)((M + 63) / 64) * ((N + 63) / 64) >= 128) return launch_dma<64, 64, BK, 2, 4>(x, w, out, gated, M, N, K, ldx, inter, K, 0, 1, st);
  return MS_UNSUPPORTED;  // too few tiles without a split of K
}

// Splits of K for the tile kernel when the caller takes partial sums and 128 x 128 tiles alone would
// not fill the chip. Up to 512 rows (large decode batches, short portions of prompts) the
// product is then bound by reading the weights, and what counts is that about 512 blocks (two per CU,
// all resident at once) share them. Matrices of up to 16 MB run as 64 x 64 tiles, K split up to 16
// ways with at least two slabs each; larger ones as 128-row tiles, split up to 8 ways with at least
// 512 k each (their partial sums weigh more: at 128 rows each split of a 4096-column product writes
// 2 MB that the consumer reads again). Measured at 96 to 512 rows and the layer shapes of the 0.6B
// and 8B models: 10 to 30 % faster than at most four splits chosen by tile count alone.
static bool tile_small_matrix(int N, int K) { return (long)N * K * 2 <= (16L << 20); }

extern "C" int ms_gemm_bf16_tile_splits(int M, int N, int K) {
  const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (tiles >= 256 && M <= 512 && (long)N * K * 2 < (128L << 20)) return 1;
  if (M > 512 && tiles * 4 < 256) {  // many rows of a narrow matrix: as many splits as fill the chip, at most 4
    int s = (int)((256 + tiles - 1) / tiles);
    if (s > 4) s = 4;
    while (s > 1 && K / s < 512) --s;
    return s;
  }
  if (M > 512) {
    // Up to four splits with at least 16 slabs each, by the time the tile shapes' model predicts plus
    // what the partial sums cost: each split writes M x N floats and the consumer reads them all, where
    // one product adds into the residual stream in place (measured about 3.5 TB/s for both).
    int best = 0;
    float least = 0.f;
    for (int sp = 1; sp <= 4; ++sp) {
      if (tiles * sp < 256 || (sp > 1 && K / sp < 16 * BK)) continue;
      float t;
      pick_tile_cols(M, N, K, sp, false, &t);
      if (sp > 1) t += (float)M * N * 4.f * (2 * sp - 1) / 3.5e6f;
      if (best == 0 || t < least) {
        least = t;
        best = sp;
      }
    }
    if (best == 0) best = tiles >= 256 ? 1 : (int)((256 + tiles - 1) / tiles);
    const int slabs = (K + BK - 1) / BK, per = (slabs + best - 1) / best;
    return (slabs + per - 1) / per;  // no empty split
  }
  if ((long)N * K * 2 >= (128L << 20)) {
    // Up to 512 rows of a large matrix with a long K: the same search over more splits. Many short
    // splits make enough 256 x 256 tiles to give every CU one (512 x 5,120 x 25,600: six parts, 240
    // tiles, 136 us against 158 for 128 x 128 tiles in three parts; a 512-token portion of the 32B shape
    // 1.5 % faster, a 256-token portion 5 %). Smaller matrices measured no gain, or lost.
    const int parts[8] = {1, 2, 3, 4, 6, 8, 12, 16};
    int best = 0;
    float least = 0.f;
    for (int c = 0; c < 8; ++c) {
      const int sp = parts[c];
      if (tiles * sp < 256 || (sp > 1 && K / sp < 8 * BK)) continue;
      float t;
      pick_tile_cols(M, N, K, sp, false, &t);
      if (sp > 1) t += (float)M * N * 4.f * (2 * sp - 1) / 3.5e6f;
      if (best == 0 || t < least) {
        least = t;
        best = sp;
      }
    }
    if (best > 0) {
      const int slabs = (K + BK - 1) / BK, per = (slabs + best - 1) / best;
      return (slabs + per - 1) / per;  // no empty split
    }
  }
  long want, most;
  if (tile_small_matrix(N, K)) {
    want = 512 / ((long)((M + 63) / 64) * ((N + 63) / 64));
    most = K / BK / 2 < 16 ? K / BK / 2 : 16;
  } else {
    want = 512 / tiles;
    most = K / 512 < 8 ? K / 512 : 8;
  }
  if (want > most) want = most;
  const int allowed[8] = {16, 12, 8, 6, 4, 3, 2, 1};
  int s = 1;
  for (int i = 0; i < 8; ++i)
    if (allowed[i] <= want) {
      s = allowed[i];
      break;
    }
  const int slabs = (K + BK - 1) / BK, per = (slabs + s - 1) / s;
  return (slabs + per - 1) / per;  // no empty split
}

// Which tile ms_gemm_bf16 (gated == 0) or the tile form of ms_gemm_bf16_gated (gated != 0, N = 2 inter) runs a
// product of these sizes with, as rows * 1000 + columns: 256256, 128064, 128128, 128160, 128192 or 64064 for the
// kernel whose slabs go straight into LDS, 0 where K or the alignment sends the product to the kernel that
// stages slabs through registers. For tests that must know which instance they have reached.
extern "C" int ms_gemm_bf16_tile_shape(int M, int N, int K, int ldx, int splits, int gated) {
  if (M <= 0 || N <= 0 || K <= 0 || splits < 1 || K % BK || ldx % 8) return 0;
  const long big = (long)((M + 127) / 128) * ((N + 127) / 128) * splits;
  if (big < 256) return 64064;
  const int cols = pick_tile_cols(M, N, K, splits, gated != 0);
  if (cols == 256) return wide_tile_offsets_fit(ldx, K) ? 256256 : 128128;
  return 128000 + cols;
}

// mode 0: C bf16 = X W^T   mode 1: C float = X W^T   mode 2: C float += X W^T
// splits > 1 (mode 1 only): C holds splits * M * N floats of partial sums, slice after slice.
extern "C" int ms_gemm_bf16(const void* X, const void* W, void* C, int mode, int M, int N, int K, int ldx, int ldc,
                            int splits, hipStream_t st) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (K <= 0 || ldx < K || ldc < N || mode < 0 || mode > 2 || splits < 1 || (splits > 1 && (mode != 1 || ldc != N)))
    return MS_BAD_ARG;
  const bf16* x = (const bf16*)X;
  const bf16* w = (const bf16*)W;
  const int k_per = ((K + splits - 1) / splits + BK - 1) / BK * BK;
  const int nz = (K + k_per - 1) / k_per;
  if (nz != splits) return MS_BAD_ARG;  // the caller sized C for `splits` slices
  const size_t stride = (size_t)M * N;
  // Large tiles when they still give every CU work; small tiles otherwise.
  const long big = (long)((M + 127) / 128) * ((N + 127) / 128) * splits;
  // Whole 64-k slabs and 16-byte aligned rows: the kernel whose slabs go straight into LDS. Of the
  // shapes tried at M = 2048 (tiles 128 or 256 wide, slabs of 32 or 64 k, 2 to 4 stages, 1 to 4 blocks
  // per CU) 128 x 128 tiles with two stages of 64 k and two blocks per CU were fastest throughout.
  if (K % BK == 0 && ldx % 8 == 0) {
    if (big >= 256)
      return launch_picked(pick_tile_cols(M, N, K, splits, false), x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
    return launch_dma<64, 64, BK, 2, 4>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride, splits, st);
  }
  if (big >= 256) {
    dim3 grid((N + 127) / 128, (M + 127) / 128, splits);
    if (grid.y > 65535) return MS_BAD_ARG;
    gemm_bf16_tile_kernel<128, 128><<<grid, 256, 0, st>>>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride);
  } else {
    dim3 grid((N + 63) / 64, (M + 63) / 64, splits);
    if (grid.y > 65535) return MS_BAD_ARG;
    gemm_bf16_tile_kernel<64, 64><<<grid, 256, 0, st>>>(x, w, C, mode, M, N, K, ldx, ldc, k_per, stride);
  }
  return launch_status();
}
