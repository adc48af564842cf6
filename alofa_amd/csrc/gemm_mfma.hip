// Matrix products whose operands are shared through LDS, bfloat16 on MFMA:
// out[m, n] = sum_k A[m, k] * W[n, k]. For prompt portions, and for few rows
// against weights so big that reading the rows again for every few weight rows
// (as the streaming kernel does) would cost more than the weights themselves.
//
// A block of four wavefronts (2 x 2) computes a tile of 64 WTM x 64 WTN outputs,
// every wave WTM x WTN tiles of v_mfma_f32_32x32x16_bf16: 128 x 128 where such
// tiles fill the chip, 64 x 64 otherwise. Per step of 64 along K the block
// stages a slab of A and of W in LDS (16-byte loads along K; rows are padded by
// 8 elements so that the fragment reads fall on distinct banks), while the next
// slabs are already on their way from memory into registers. Accumulation is
// float; each output element has one accumulator that takes the products in
// ascending k, whatever M is.
//
// Where even the small tiles are too few for the chip (few rows, few columns, a
// long K), K is shared out among blocks as well: every block leaves its partial tile
// in the workspace, and the one that arrives last adds them in a fixed order and
// runs the epilogue (the protocol of the streaming kernel, see there).
//
// Operand layout of the instruction, lane l: A holds row l % 32 and B column
// l % 32, both the reduction indices 8 * (l / 32) .. + 7 of the 16; D holds
// column l % 32 and, in acc[i], row 8 * (i / 4) + 4 * (l / 32) + i % 4.
//
// Epilogues: store (+ bias), add to the float residual stream, and SwiGLU, for
// which a block computes the gate and the up product of the same columns (its
// W slab holds as many rows of each) and writes silu(gate) * up.
#include "common.h"

#include <cstdlib>

namespace alofa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum MfmaEpilogue : int { kMfStore = 0, kMfResidual = 1, kMfSwiglu = 2, kMfArgmax = 3 };

constexpr int TK = 64, PAD = 8;
constexpr int kRow = TK + PAD;  // LDS row length in elements

// Which tile a block computes. The chip is eight dies, each with an L2 of its own, and blocks go to the
// dies in turn (block i to die i % 8). Dealt out row by row, every die computes tiles from all over the
// output and pulls all of A and all of W through its L2: fine while both fit there, and measured a few
// percent faster then than the path below; with operands beyond the L2s (projections of 7B-sized models
// and up) it costs up to a fifth of the time. For those (by_die) the tiles are numbered along a path that
// stays within squares of 8 x 8 tiles (8 tile rows at a time, column by column), every die takes one
// contiguous stretch of the path, and the blocks resident on a die together share a handful of A and W
// panels. With K shared out, the shares are the slowest index (blocks of different shares have nothing
// in common).
struct TilePlace {
  int bm, bn, share;
};
__device__ __forceinline__ TilePlace place_tile(int block, int tiles_m, int tiles_n, int shares, bool by_die) {
  constexpr int kDies = 8, kGroup = 8;
  const int tiles = tiles_m * tiles_n, total = tiles * shares;
  if (!by_die) return {block % tiles / tiles_n, block % tiles_n, block / tiles};
  const int die = block % kDies, local = block / kDies;
  const int step = die * (total / kDies) + min(die, total % kDies) + local;   // dies before this one hold that many blocks
  const int t = step % tiles;
  const int per_group = kGroup * tiles_n, first_m = (t / per_group) * kGroup, within = t % per_group;
  const int rows = min(tiles_m - first_m, kGroup);
  return {first_m + within % rows, within / rows, step / tiles};
}

// Instead of the outputs, a wave leaves per row the highest of its columns and that column's number (the lowest
// among equals): candidate 2 bn + wn of `parts` per row, values at out[m * parts + ..], column numbers as int32
// behind the M * parts values. A column past N is no candidate (its number reads as INT_MAX).
template <int WTM, int WTN>
__device__ __forceinline__ void tile_argmax(f32x16 (&acc)[WTM][WTN], float* __restrict__ out, int parts, int M, int N, int m0, int n0,
                                            int bn, int wm, int wn, int lane) {
  const int col = lane % 32, half = lane / 32;
  int32_t* numbers = reinterpret_cast<int32_t*>(out + static_cast<int64_t>(M) * parts);
#pragma unroll
  for (int i = 0; i < WTM; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      if (m0 + wm * 32 * WTM + i * 32 + 8 * (e / 4) >= M) continue;     // (uniform over the wave) rows past M: with 8 rows, 4 of a wave's 16 registers count
      float bv = -3.402823466e+38f;
      int bi = 0x7fffffff;
#pragma unroll
      for (int j = 0; j < WTN; ++j) {      // ascending columns: an equal value further right does not take over
        const int n = n0 + wn * 32 * WTN + j * 32 + col;
        const float v = acc[i][j][e];
        if (n < N && v > bv) { bv = v; bi = n; }
      }
#pragma unroll
      for (int off = 16; off > 0; off >>= 1) {     // the 32 lanes that hold this row's columns
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
      }
      const int m = m0 + wm * 32 * WTM + i * 32 + 8 * (e / 4) + 4 * half + e % 4;
      if (col == 0 && m < M) {
        out[static_cast<int64_t>(m) * parts + 2 * bn + wn] = bv;
        numbers[static_cast<int64_t>(m) * parts + 2 * bn + wn] = bi;
      }
    }
  }
}

// What a wave does with its finished tiles (WTM x WTN of 32 x 32, the block's tile at m0, n0 of the output).
template <int kEpilogue, typename TO, int WTM, int WTN>
__device__ __forceinline__ void tile_epilogue(f32x16 (&acc)[WTM][WTN], TO* __restrict__ out, int64_t ldo,
                                              const float* __restrict__ bias, int M, int N, int m0, int n0, int wm, int wn, int lane) {
  constexpr int kGateTiles = WTN / 2;
  const int col = lane % 32, row_base = (lane / 32) * 4;
  constexpr int kOutTiles = (kEpilogue == kMfSwiglu) ? kGateTiles : WTN;
#pragma unroll
  for (int i = 0; i < WTM; ++i) {
#pragma unroll
    for (int j = 0; j < kOutTiles; ++j) {
      const int n = n0 + wn * 32 * kOutTiles + j * 32 + col;
      if (n >= N) continue;
      const float b = (bias && kEpilogue == kMfStore) ? bias[n] : 0.f;
      const int m_first = m0 + wm * 32 * WTM + i * 32 + row_base;      // element e: row m_first + 8 * (e / 4) + e % 4
      TO* column = out + n;
      float old[16];
      if (kEpilogue == kMfResidual) {      // all sixteen old values set out before any is needed
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m_first + 8 * (e / 4) + e % 4;
          old[e] = m < M ? load_f32(column + static_cast<int64_t>(m) * ldo) : 0.f;
        }
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m_first + 8 * (e / 4) + e % 4;
        if (m >= M) continue;
        TO* dst = column + static_cast<int64_t>(m) * ldo;
        if (kEpilogue == kMfStore) {
          store_f32(dst, acc[i][j][e] + b);
        } else if (kEpilogue == kMfResidual) {
          store_f32(dst, old[e] + acc[i][j][e]);
        } else {
          const float g = acc[i][j][e];
          store_f32(dst, g / (1.f + __expf(-g)) * acc[i][(j + kGateTiles) % WTN][e]);
        }
      }
    }
  }
}

// WTM, WTN: MFMA tiles per wave along m and along n; the block tile is 64 WTM x 64 WTN.
// PF: slabs on their way from memory while another is being multiplied.
// kSplitK: a block takes a share of K; the shares meet in the workspace (see below).
template <int kEpilogue, typename TO, int WTM, int WTN, int PF, bool kSplitK>
__global__ void __launch_bounds__(256) gemm_mfma_kernel(TO* __restrict__ out, int64_t ldo,
                                                        const bf16_t* __restrict__ A, int64_t lda,
                                                        const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
                                                        int64_t ldw, const float* __restrict__ bias, int M, int N,
                                                        int K_all, int tiles_m, int tiles_n, int shares,
                                                        float* __restrict__ ws, int* __restrict__ counters, int by_die) {
  constexpr int TM = 64 * WTM, TN = 64 * WTN;
  // swiglu: the first half of a wave's column tiles are gate columns, the second half the up columns of the same outputs
  constexpr int kGateTiles = WTN / 2;
  static_assert(kEpilogue != kMfSwiglu || WTN % 2 == 0, "the swiglu epilogue needs an even number of column tiles per wave");
  __shared__ int last_block;
  const TilePlace place = place_tile(blockIdx.x, tiles_m, tiles_n, shares, by_die != 0);
  // this block's share of K: slabs [k_begin, K)
  int k_begin = 0, K = K_all;
  if (kSplitK) {
    const int slabs = (K_all + TK - 1) / TK, per_split = (slabs + shares - 1) / shares;
    k_begin = place.share * per_split * TK;
    K = min(K_all, k_begin + per_split * TK);
  }
  __shared__ __attribute__((aligned(16))) bf16_t As[TM * kRow];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[TN * kRow];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = wave / 2, wn = wave % 2;
  constexpr int kOutCols = (kEpilogue == kMfSwiglu) ? TN / 2 : TN;
  const int m0 = place.bm * TM, n0 = place.bn * kOutCols;

  // global -> register staging: 8 chunks of 16 bytes per slab row; a thread takes row (tid + 256 j) / 8
  constexpr int NCA = WTM * 2, NCW = WTN * 2;
  const int c_k = (tid % 8) * 8;
  const bf16_t* a_src[NCA];
  const bf16_t* w_src[NCW];
  bool a_ok[NCA], w_ok[NCW];
#pragma unroll
  for (int j = 0; j < NCA; ++j) {
    const int m = m0 + (tid + 256 * j) / 8;
    a_ok[j] = m < M;
    a_src[j] = A + static_cast<int64_t>(a_ok[j] ? m : 0) * lda + c_k;
  }
#pragma unroll
  for (int j = 0; j < NCW; ++j) {
    const int row = (tid + 256 * j) / 8;
    int n = n0 + row;
    const bf16_t* base = W;
    if (kEpilogue == kMfSwiglu && row >= TN / 2) {  // slab rows below TN / 2: gate rows n0 ..; the others: up rows of the same columns
      n = n0 + row - TN / 2;
      base = W2;
    }
    w_ok[j] = n < N;
    w_src[j] = base + static_cast<int64_t>(w_ok[j] ? n : 0) * ldw + c_k;
  }

  f32x16 acc[WTM][WTN];
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int j = 0; j < WTN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  uint4 a_reg[PF][NCA], w_reg[PF][NCW];
  auto fetch = [&](uint4 (&a)[NCA], uint4 (&w)[NCW], int k0) {
    // Every lane issues every load (from the row's start where the values are not wanted; zeros are put in
    // their place at staging): with loads that are always issued the compiler can count them and wait for
    // the oldest slab only, so that the later ones stay on their way.
    const int koff = (k0 + c_k < K) ? k0 : -c_k;
#pragma unroll
    for (int j = 0; j < NCA; ++j) a[j] = *reinterpret_cast<const uint4*>(a_src[j] + koff);
#pragma unroll
    for (int j = 0; j < NCW; ++j) w[j] = *reinterpret_cast<const uint4*>(w_src[j] + koff);
  };
  auto stage = [&](const uint4 (&a)[NCA], const uint4 (&w)[NCW], int k0) {
    const bool k_ok = k0 + c_k < K;
    const int first = (tid / 8) * kRow + c_k;    // chunk j lies 32 slab rows further on
#pragma unroll
    for (int j = 0; j < NCA; ++j) {
      const uint32_t ka = 0u - static_cast<uint32_t>(k_ok && a_ok[j]);   // all ones or zero
      *reinterpret_cast<uint4*>(&As[first + j * 32 * kRow]) = make_uint4(a[j].x & ka, a[j].y & ka, a[j].z & ka, a[j].w & ka);
    }
#pragma unroll
    for (int j = 0; j < NCW; ++j) {
      const uint32_t kw = 0u - static_cast<uint32_t>(k_ok && w_ok[j]);
      *reinterpret_cast<uint4*>(&Ws[first + j * 32 * kRow]) = make_uint4(w[j].x & kw, w[j].y & kw, w[j].z & kw, w[j].w & kw);
    }
  };

  // rows of the fragments this lane reads
  const int frag_row = lane % 32, frag_k = (lane / 32) * 8;
  int a_off[WTM], w_off[WTN];
#pragma unroll
  for (int i = 0; i < WTM; ++i) a_off[i] = (wm * 32 * WTM + i * 32 + frag_row) * kRow + frag_k;
#pragma unroll
  for (int j = 0; j < WTN; ++j) {
    int row = wn * 32 * WTN + j * 32 + frag_row;
    if (kEpilogue == kMfSwiglu)   // this wave's 32 kGateTiles output columns: their gate rows, then their up rows
      row = (j < kGateTiles) ? wn * 32 * kGateTiles + j * 32 + frag_row : TN / 2 + wn * 32 * kGateTiles + (j - kGateTiles) * 32 + frag_row;
    w_off[j] = row * kRow + frag_k;
  }
  auto multiply = [&]() {
#pragma unroll
    for (int ks = 0; ks < TK; ks += 16) {
      bf16x8 a[WTM], w[WTN];
#pragma unroll
      for (int i = 0; i < WTM; ++i) a[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&As[a_off[i] + ks]));
#pragma unroll
      for (int j = 0; j < WTN; ++j) w[j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Ws[w_off[j] + ks]));
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WTN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], w[j], acc[i][j], 0, 0, 0);
    }
  };

  // The slabs set out in the order in which they are needed, and the compiler may not change it: the
  // loads of a wave complete in order, and the wait for slab p must leave the later ones on their way.
#pragma unroll
  for (int p = 0; p < PF; ++p) {
    fetch(a_reg[p], w_reg[p], k_begin + p * TK);
    __builtin_amdgcn_sched_barrier(0);
  }
  // Whole rounds of PF slabs first, without a branch inside: a slab that could be skipped would make the
  // compiler wait for every load at the next one (on the path past it the loads just issued are the
  // youngest). The last, partial round follows the loop and sets no further loads out.
  int k0 = k_begin;
  for (; k0 + (PF - 1) * TK < K; k0 += PF * TK) {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      __builtin_amdgcn_sched_barrier(0);   // (nor may slab p's staging, and with it the wait for its loads, move up into the step before)
      __syncthreads();        // the previous slab has been read by every wave
      stage(a_reg[p], w_reg[p], k0 + p * TK);
      __syncthreads();
      fetch(a_reg[p], w_reg[p], k0 + (p + PF) * TK);
      multiply();
    }
  }
#pragma unroll
  for (int p = 0; p < PF - 1; ++p) {
    if (k0 + p * TK < K) {    // uniform over the block
      __syncthreads();
      stage(a_reg[p], w_reg[p], k0 + p * TK);
      __syncthreads();
      multiply();
    }
  }

  if (kSplitK) {
    // The shares of K meet in the workspace: every block leaves its tile there (at device scope: written
    // through to memory, where blocks on every die find it) and is counted once every wave's stores have
    // been acknowledged; the block counted last adds the tiles in split order, so the sum is the same on
    // every run, goes on to the epilogue and puts the counter back to zero.
    const int splits = shares, tile_id = place.bm * tiles_n + place.bn;
    constexpr int kTileFloats = WTM * WTN * 16 * 256;
    float* mine = ws + (static_cast<int64_t>(tile_id) * splits + place.share) * kTileFloats;
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WTN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          __hip_atomic_store(mine + ((i * WTN + j) * 16 + e) * 256 + tid, acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      const int arrived = atomicAdd(&counters[tile_id], 1);
      last_block = arrived == splits - 1;
      if (last_block) atomicExch(&counters[tile_id], 0);
    }
    __syncthreads();
    if (!last_block) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const float* parts = ws + static_cast<int64_t>(tile_id) * splits * kTileFloats;
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WTN; ++j) {
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        for (int sp0 = 0; sp0 < splits; sp0 += 4) {     // four shares' loads on their way together; added in the shares' order
          float part[4][16];
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < 16; ++e)
              part[u][e] = __hip_atomic_load(parts + static_cast<int64_t>(min(sp0 + u, splits - 1)) * kTileFloats + ((i * WTN + j) * 16 + e) * 256 + tid,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (sp0 + u < splits) {
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[i][j][e] += part[u][e];
            }
        }
      }
  }

  if constexpr (kEpilogue == kMfArgmax) {
    tile_argmax<WTM, WTN>(acc, out, static_cast<int>(ldo), M, N, m0, n0, place.bn, wm, wn, lane);
    return;
  } else {
    tile_epilogue<kEpilogue, TO, WTM, WTN>(acc, out, ldo, bias, M, N, m0, n0, wm, wn, lane);
  }
}

// The same product with the slabs brought from memory straight into LDS (global_load_lds_dwordx4: every lane's
// 16 bytes land at consecutive LDS addresses, 1 KB per wave and instruction, no registers and no LDS writes in
// between) into a ring of S slabs, S - 1 of them on their way while one is multiplied. For K a multiple of 64; with
// kSplitK a block takes a share of the slabs and the shares meet in the workspace as above. Which products take it:
// see launch_mfma.
// A slab is 64 WTM rows of A and 64 WTN rows of W, 128 bytes each, unpadded; the eight 16-byte chunks of a row are
// permuted by the row's number (chunk c of row r lies at place c ^ swz(r)), which the lane that fetches place p
// of row r undoes by fetching chunk p ^ swz(r), so that the 16 or 32 rows whose fragments are read together
// fall on distinct banks.
// Rows beyond M or N are fetched from the last valid row (their results are never stored).
__device__ __forceinline__ int swz(int r) { return (r & 7) ^ ((r >> 3) & 1); }

// kSplitK = 2: a block leaves its share's sums as they are, tile by tile, in part `share` of `out` (float
// [shares, M, ldo]); a second kernel (split_sum_kernel) adds the parts and runs the epilogue.
template <int kEpilogue, typename TO, int WTM, int WTN, int S, int kSplitK = 0>
__global__ void __launch_bounds__(256) gemm_dma_kernel(TO* __restrict__ out, int64_t ldo, const bf16_t* __restrict__ A, int64_t lda,
                                                       const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2, int64_t ldw,
                                                       const float* __restrict__ bias, int M, int N, int K, int tiles_m,
                                                       int tiles_n, int by_die, int shares = 1, float* __restrict__ ws = nullptr,
                                                       int* __restrict__ counters = nullptr, int own = 0) {
  constexpr int TM = 64 * WTM, TN = 64 * WTN;
  constexpr int kGateTiles = WTN / 2;
  // (swiglu with WTN = 1: the waves of column 0 take 32 gate columns, those of column 1 the up columns of the same
  // outputs, and the two meet in LDS after the last slab)
  static_assert(kEpilogue != kMfSwiglu || WTN % 2 == 0 || WTN == 1, "the swiglu epilogue needs an even number of column tiles per wave, or one");
  constexpr int kRows = TM + TN;               // slab rows: A's, then W's
  constexpr int kStageBytes = kRows * 128;
  constexpr int kLoads = kRows / 32;           // fetch instructions per wave and slab (each brings eight rows)
  __shared__ __attribute__((aligned(1024))) char ring[S * kStageBytes];
  __shared__ int last_block;
  const TilePlace place = place_tile(blockIdx.x, tiles_m, tiles_n, kSplitK ? shares : 1, by_die != 0);
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = wave / 2, wn = wave % 2;
  constexpr int kOutCols = (kEpilogue == kMfSwiglu) ? TN / 2 : TN;
  // (own: the output columns a block owns of those its tile holds, all of them if 0: see launch_dma. The columns
  // beyond are fetched from the last owned one, which costs no memory traffic, and never stored.)
  const int owned = own > 0 ? own : kOutCols;
  const int m0 = place.bm * TM, n0 = place.bn * owned;
  const int n_end = min(N, n0 + owned);

  // what this lane fetches: instruction j of this wave brings slab rows 8 (4 j + wave) .. + 7, lane l place l % 8 of row l / 8
  const bf16_t* src[kLoads];
#pragma unroll
  for (int j = 0; j < kLoads; ++j) {
    const int r = 8 * (4 * j + wave) + lane / 8, c = (lane % 8) ^ swz(r);
    if (r < TM) {
      src[j] = A + static_cast<int64_t>(min(m0 + r, M - 1)) * lda + c * 8;
    } else {
      const int row = r - TM;
      int n = n0 + row;
      const bf16_t* base = W;
      if (kEpilogue == kMfSwiglu && row >= TN / 2) {   // slab rows below TN / 2: gate rows n0 ..; the others: up rows of the same columns
        n = n0 + row - TN / 2;
        base = W2;
      }
      src[j] = base + static_cast<int64_t>(min(n, n_end - 1)) * ldw + c * 8;
    }
  }
  // The fetches are written out as instructions: the compiler, which cannot tell the ring's slabs apart, would wait
  // for every fetch on its way before any read from LDS, and the slabs set out ahead would be waited for at once.
  // (M0 holds the LDS address of the wave's first lane; the instruction adds 16 bytes per lane.)
  const unsigned ring_at = static_cast<unsigned>(reinterpret_cast<uintptr_t>(ring));
  auto fetch = [&](int slab) {     // uniform over the block
    const unsigned stage = ring_at + (slab % S) * kStageBytes + wave * 1024;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const bf16_t* from = src[j] + static_cast<int64_t>(slab) * TK;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   :: "s"(__builtin_amdgcn_readfirstlane(stage + j * 4096)), "v"(from), "r"(ring) : "memory", "m0");
    }
  };

  f32x16 acc[WTM][WTN];
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int j = 0; j < WTN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // fragments: lane l reads row l % 32 of its 32-row group, chunk 2 q + l / 32 in step q of the slab's four
  const int sw = swz(lane % 32), half = lane / 32;
  const int a_row = (wm * 32 * WTM + lane % 32) * 128;
  const int w_row = (TM + wn * 32 * (kEpilogue == kMfSwiglu ? (WTN == 1 ? 1 : kGateTiles) : WTN) + lane % 32) * 128;
  int place_of[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) place_of[q] = ((2 * q + half) ^ sw) * 16;
  auto w_group = [&](int j) {      // byte offset of this wave's j-th 32-row group of W within the slab's W rows
    if (kEpilogue == kMfSwiglu && WTN == 1) return 0;
    if (kEpilogue == kMfSwiglu) return (j < kGateTiles ? j * 32 : TN / 2 + (j - kGateTiles) * 32) * 128;
    return j * 32 * 128;
  };

  // (with K shared out this block takes the slabs first .. slabs - 1 of all)
  const int all_slabs = K / TK, per_share = kSplitK ? (all_slabs + shares - 1) / shares : all_slabs;
  const int first = kSplitK ? place.share * per_share : 0;
  const int slabs = min(first + per_share, all_slabs);
  bf16x8 a[4][WTM], w[4][WTN];
  auto read = [&](int slab) {
    const char* stage = ring + (slab % S) * kStageBytes;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int i = 0; i < WTM; ++i) a[q][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(stage + a_row + i * 32 * 128 + place_of[q]));
#pragma unroll
      for (int j = 0; j < WTN; ++j) w[q][j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(stage + w_row + w_group(j) + place_of[q]));
    }
  };
  auto multiply = [&]() {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WTN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[q][i], w[q][j], acc[i][j], 0, 0, 0);
  };

  // Slab k + S - 1 is set out once every wave has read slab k - 1 (whose place it takes), i.e. after the barrier
  // of step k, and has the multiplications of S - 1 steps to arrive. A wave waits for its own fetches of slab k
  // (the S - 2 slabs behind it stay on their way) before the barrier; behind the barrier all of the slab is there.
  constexpr int kLead = S - 1;
#pragma unroll
  for (int p = 0; p < kLead; ++p)
    if (first + p < slabs) fetch(first + p);
  int k = first;
  for (; k + kLead < slabs; ++k) {
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kLoads * (kLead - 1)) : "memory");
    __syncthreads();
    read(k);
    fetch(k + kLead);
    multiply();
  }
  for (; k < slabs; ++k) {      // nothing more to set out: the last slabs as they come
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    read(k);
    multiply();
  }
  if constexpr (kEpilogue == kMfSwiglu && WTN == 1) {
    __syncthreads();      // every wave has read the last slab: the ring is free
    float* meet = reinterpret_cast<float*>(ring);     // [wm][i][e][lane]
    if (wn == 1) {
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) meet[((wm * WTM + i) * 16 + e) * 64 + lane] = acc[i][0][e];
    }
    __syncthreads();
    if (wn == 0) {
      const int n = n0 + lane % 32;
#pragma unroll
      for (int i = 0; i < WTM; ++i) {
        const int m_first = m0 + wm * 32 * WTM + i * 32 + (lane / 32) * 4;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m_first + 8 * (e / 4) + e % 4;
          const float g = acc[i][0][e], up = meet[((wm * WTM + i) * 16 + e) * 64 + lane];
          if (m < M && n < n_end) store_f32(out + static_cast<int64_t>(m) * ldo + n, g / (1.f + __expf(-g)) * up);
        }
      }
    }
    return;
  }
  if constexpr (kSplitK == 2) {
    static_assert(kEpilogue == kMfStore && sizeof(TO) == 4, "parts of a sum are stored as float");
    tile_epilogue<kEpilogue, TO, WTM, WTN>(acc, out + static_cast<int64_t>(place.share) * M * ldo, ldo, nullptr, M, N, m0, n0, wm, wn, lane);
    return;
  }
  if constexpr (kSplitK == 1) {
    // the shares of K meet in the workspace, as in the kernel above
    const int tile_id = place.bm * tiles_n + place.bn;
    constexpr int kTileFloats = WTM * WTN * 16 * 256;
    float* mine = ws + (static_cast<int64_t>(tile_id) * shares + place.share) * kTileFloats;
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WTN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          __hip_atomic_store(mine + ((i * WTN + j) * 16 + e) * 256 + tid, acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      const int arrived = atomicAdd(&counters[tile_id], 1);
      last_block = arrived == shares - 1;
      if (last_block) atomicExch(&counters[tile_id], 0);
    }
    __syncthreads();
    if (!last_block) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const float* parts = ws + static_cast<int64_t>(tile_id) * shares * kTileFloats;
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WTN; ++j) {
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        for (int sp0 = 0; sp0 < shares; sp0 += 4) {     // four shares' loads on their way together; added in the shares' order
          float part[4][16];
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < 16; ++e)
              part[u][e] = __hip_atomic_load(parts + static_cast<int64_t>(min(sp0 + u, shares - 1)) * kTileFloats + ((i * WTN + j) * 16 + e) * 256 + tid,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (sp0 + u < shares) {
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[i][j][e] += part[u][e];
            }
        }
      }
  }
  tile_epilogue<kEpilogue, TO, WTM, WTN>(acc, out, ldo, bias, M, n_end, m0, n0, wm, wn, lane);
}

// The tiled product for many rows against a wide matrix: eight waves (WM x WN) on a tile of TM x TN outputs, slabs of 32
// along K straight from memory into a ring of S in LDS. Against the four waves and slabs of 64 above: a wave's share of
// a slab is small enough (a tile of 256 x 256 in 128 KB of ring) for two waves a SIMD, which fill one another's waits
// at the barrier and for LDS, and a slab carries twice the products per byte fetched. The sums are the same numbers in
// the same order as in the kernels above (one accumulator an output, ascending k). K a multiple of 32.
// A slab is TM rows of A and TN rows of W, 64 bytes each; the four 16-byte chunks of a row are permuted by the row's
// number (chunk c of row r lies at place c ^ ((r >> 2) & 3)), so that the sixteen rows whose fragments a quarter of a
// wave reads together fall on distinct banks. kMfSwiglu: the slab's W rows are TN / 2 gate rows, then the up rows of the
// same columns, and a wave holds gate and up of the same columns.
__device__ __forceinline__ int swz32(int r) { return (r >> 2) & 3; }

template <int kEpilogue, typename TO, int TM, int TN, int WM, int WN, int S>
__global__ void __launch_bounds__(64 * WM * WN) gemm_wide_kernel(TO* __restrict__ out, int64_t ldo, const bf16_t* __restrict__ A, int64_t lda,
                                                                 const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2, int64_t ldw,
                                                                 const float* __restrict__ bias, int M, int N, int K, int tiles_m, int tiles_n) {
  constexpr int kSlabK = 32, kRows = TM + TN, kStageBytes = kRows * 64, kWaves = WM * WN;
  constexpr int kLoads = kRows / 16 / kWaves;        // fetch instructions per wave and slab (each brings sixteen rows)
  constexpr int TI = TM / 32 / WM, TJ = TN / 32 / WN;   // 32 x 32 tiles a wave
  static_assert(kRows % (16 * kWaves) == 0 && TM % (32 * WM) == 0 && TN % (32 * WN) == 0, "the tile must divide among the waves");
  static_assert(kEpilogue != kMfSwiglu || TJ % 2 == 0, "the swiglu epilogue needs gate and up tiles in every wave");
  constexpr int kGateTiles = TJ / 2;
  __shared__ __attribute__((aligned(1024))) char ring[S * kStageBytes];
  const TilePlace place = place_tile(blockIdx.x, tiles_m, tiles_n, 1, true);
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = wave / WN, wn = wave % WN;
  constexpr int kOutCols = (kEpilogue == kMfSwiglu) ? TN / 2 : TN;
  const int m0 = place.bm * TM, n0 = place.bn * kOutCols;

  // what this lane fetches: instruction j of this wave brings slab rows 16 (kWaves j + wave) .. + 15, lane l place l % 4 of row l / 4
  const bf16_t* src[kLoads];
#pragma unroll
  for (int j = 0; j < kLoads; ++j) {
    const int r = 16 * (kWaves * j + wave) + lane / 4, c = (lane % 4) ^ swz32(r);
    if (r < TM) {
      src[j] = A + static_cast<int64_t>(min(m0 + r, M - 1)) * lda + c * 8;
    } else {
      const int row = r - TM;
      int n = n0 + row;
      const bf16_t* base = W;
      if (kEpilogue == kMfSwiglu && row >= TN / 2) {
        n = n0 + row - TN / 2;
        base = W2;
      }
      src[j] = base + static_cast<int64_t>(min(n, N - 1)) * ldw + c * 8;
    }
  }
  const unsigned ring_at = static_cast<unsigned>(reinterpret_cast<uintptr_t>(ring));
  auto fetch = [&](int slab) {     // uniform over the block
    const unsigned stage = ring_at + (slab % S) * kStageBytes + wave * 1024;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const bf16_t* from = src[j] + static_cast<int64_t>(slab) * kSlabK;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   :: "s"(__builtin_amdgcn_readfirstlane(stage + j * kWaves * 1024)), "v"(from), "r"(ring) : "memory", "m0");
    }
  };

  f32x16 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // fragments: lane l reads row l % 32 of its 32-row group, chunk 2 q + l / 32 in step q of the slab's two
  const int sw = swz32(lane % 32), half = lane / 32;
  const int a_row = (wm * 32 * TI + lane % 32) * 64;
  const int w_row = (TM + lane % 32) * 64;
  int place_of[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) place_of[q] = ((2 * q + half) ^ sw) * 16;
  auto w_group = [&](int j) {      // byte offset of this wave's j-th 32-row group within the slab's W rows
    if (kEpilogue == kMfSwiglu) return ((j < kGateTiles ? 0 : TN / 2) + (wn * kGateTiles + j % kGateTiles) * 32) * 64;
    return (wn * TJ + j) * 32 * 64;
  };
  auto step = [&](int slab) {
    const char* stage = ring + (slab % S) * kStageBytes;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      bf16x8 a[TI], w[TJ];
#pragma unroll
      for (int i = 0; i < TI; ++i) a[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(stage + a_row + i * 32 * 64 + place_of[q]));
#pragma unroll
      for (int j = 0; j < TJ; ++j) w[j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(stage + w_row + w_group(j) + place_of[q]));
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], w[j], acc[i][j], 0, 0, 0);
    }
  };

  // Slab k + S - 1 takes the place of slab k - 1, which every wave has read before the barrier of step k; a wave waits
  // for its own fetches of slab k (the S - 2 slabs behind it stay on their way) before that barrier.
  const int slabs = K / kSlabK;
  constexpr int kLead = S - 1;
#pragma unroll
  for (int p = 0; p < kLead; ++p)
    if (p < slabs) fetch(p);
  int k = 0;
  for (; k + kLead < slabs; ++k) {
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kLoads * (kLead - 1)) : "memory");
    __syncthreads();
    fetch(k + kLead);
    step(k);
  }
  for (; k < slabs; ++k) {      // nothing more to set out: the last slabs as they come
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    step(k);
  }
  tile_epilogue<kEpilogue, TO, TI, TJ>(acc, out, ldo, bias, M, N, m0, n0, wm, wn, lane);
}

template <int kEpilogue, typename TO, int TM, int TN, int WM, int WN, int S>
static int launch_wide(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, int64_t ldw, const float* bias, int M, int N, int K,
                       hipStream_t stream, const void* W2 = nullptr) {
  constexpr int kOutCols = (kEpilogue == kMfSwiglu) ? TN / 2 : TN;
  const int tiles_n = (N + kOutCols - 1) / kOutCols, tiles_m = (M + TM - 1) / TM;
  gemm_wide_kernel<kEpilogue, TO, TM, TN, WM, WN, S><<<tiles_n * tiles_m, 64 * WM * WN, 0, stream>>>(
      static_cast<TO*>(out), ldo, static_cast<const bf16_t*>(A), lda, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2), ldw, bias, M, N, K,
      tiles_m, tiles_n);
  return 0;
}

// Where the tiles of 256 x 256 with eight waves are the tiled product's choice: many rows against a long K, and so many
// tiles that their rounds of one a compute unit are at least four fifths full. Measured against the forms below
// (2,048 rows, us): gate/up + SwiGLU of the 7B sizes 524 against 586, of the 32B sizes 1,043 against 1,169 (4,096 rows:
// 2,086 against 2,268; 256 rows, 216 tiles: 174 against 254); 7,168 x 5,120 150 against 183 (4,096 rows: 293 against
// 350); 3,584 x 3,584 at 4,096 rows 116 against 142, 3,584 x 18,944 538 against 592. With rounds less full the forms
// below stay ahead (7B gate/up at 512 rows, 296 tiles: 210 against 176; 5,120 x 27,648 at 4,096 rows, 320 tiles: 1,507
// against 1,285), and so they do with a short K (0.5B gate/up at 2,048 rows 60.6 against 46.3).
template <int kEpilogue>
static bool wide_pays(int M, int N, int K) {
  static const bool switched_off = [] { const char* e = getenv("ALOFA_WIDE_TILES"); return e != nullptr && e[0] == '0'; }();     // (for measurements)
  if (switched_off || M <= 128 || K % 32 != 0 || K < 2048) return false;
  constexpr int kOutCols = (kEpilogue == kMfSwiglu) ? 128 : 256;
  const int64_t tiles = static_cast<int64_t>((M + 255) / 256) * ((N + kOutCols - 1) / kOutCols), units = compute_units();
  const int64_t rounds = (tiles + units - 1) / units;
  return tiles * 5 >= rounds * units * 4;
}

template <int kEpilogue, typename TO, int WTM, int WTN, int PF, bool kSplitK>
static int launch_tile(int tiles_n, int tiles_m, int shares, void* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                       const float* bias, int M, int N, int K, hipStream_t stream) {
  const Workspace& g_ws = workspace();
  if (kSplitK) {   // the partial tiles and the counters of all tiles must lie within the workspace: checked here, whatever chose the shares
    const int64_t tiles = static_cast<int64_t>(tiles_n) * tiles_m;
    ALOFA_REQUIRE(g_ws.tiles != nullptr && tiles <= g_ws.n_counters && tiles * shares * (WTM * WTN * 16 * 256) <= g_ws.tile_floats,
                  "gemm_mfma: %lld tiles in %d shares of K do not fit the workspace", static_cast<long long>(tiles), shares);
  }
  // operands beyond what the eight L2s hold together (4 MB each)
  const int w_rows = (kEpilogue == kMfSwiglu) ? 2 * N : N;
  const int by_die = (static_cast<int64_t>(M) + w_rows) * K * 2 > (32 << 20);
  gemm_mfma_kernel<kEpilogue, TO, WTM, WTN, PF, kSplitK><<<tiles_n * tiles_m * shares, 256, 0, stream>>>(
      static_cast<TO*>(out), ldo, static_cast<const bf16_t*>(A), lda, static_cast<const bf16_t*>(W),
      static_cast<const bf16_t*>(W2), ldw, bias, M, N, K, tiles_m, tiles_n, shares, kSplitK ? g_ws.tiles : nullptr,
      kSplitK ? g_ws.counters : nullptr, by_die);
  return 0;
}

template <int kEpilogue, typename TO, int WTM, int WTN, int S>
static int launch_dma_shared(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, int64_t ldw, const float* bias, int M, int N, int K,
                             int shares, hipStream_t stream) {
  const int tiles_n = (N + 64 * WTN - 1) / (64 * WTN), tiles_m = (M + 64 * WTM - 1) / (64 * WTM);
  const Workspace& g_ws = workspace();
  const int64_t tiles = static_cast<int64_t>(tiles_n) * tiles_m;
  ALOFA_REQUIRE(g_ws.tiles != nullptr && tiles <= g_ws.n_counters && tiles * shares * (WTM * WTN * 16 * 256) <= g_ws.tile_floats,
                "gemm_mfma: %lld tiles in %d shares of K do not fit the workspace", static_cast<long long>(tiles), shares);
  gemm_dma_kernel<kEpilogue, TO, WTM, WTN, S, 1><<<tiles_n * tiles_m * shares, 256, 0, stream>>>(
      static_cast<TO*>(out), ldo, static_cast<const bf16_t*>(A), lda, static_cast<const bf16_t*>(W), nullptr, ldw, bias, M, N, K,
      tiles_m, tiles_n, 1, shares, g_ws.tiles, g_ws.counters);
  return 0;
}

// out = epilogue(sum over the parts, in their order) for parts [shares, M, N] of float; four columns a thread.
template <int kEpilogue, typename TO>
__global__ void __launch_bounds__(256) split_sum_kernel(TO* __restrict__ out, int64_t ldo, const float* __restrict__ parts, int shares,
                                                        const float* __restrict__ bias, int M, int N) {
  const int groups = N / 4;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(M) * groups) return;
  const int m = static_cast<int>(idx / groups), n = static_cast<int>(idx % groups) * 4;
  const float* src = parts + static_cast<int64_t>(m) * N + n;
  // (eight parts' loads on their way together: the parts come from memory, one after the other they are waited for one by one)
  float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
  const int64_t part = static_cast<int64_t>(M) * N;
  for (int s0 = 0; s0 < shares; s0 += 8) {
    float4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const float4*>(src + min(s0 + i, shares - 1) * part);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (s0 + i < shares) { sum.x += v[i].x; sum.y += v[i].y; sum.z += v[i].z; sum.w += v[i].w; }
  }
  TO* dst = out + static_cast<int64_t>(m) * ldo + n;
  if constexpr (kEpilogue == kMfResidual) {
    dst[0] += sum.x; dst[1] += sum.y; dst[2] += sum.z; dst[3] += sum.w;
  } else {
    if (bias != nullptr) { sum.x += bias[n]; sum.y += bias[n + 1]; sum.z += bias[n + 2]; sum.w += bias[n + 3]; }
    store_f32(dst, sum.x); store_f32(dst + 1, sum.y); store_f32(dst + 2, sum.z); store_f32(dst + 3, sum.w);
  }
}

// An RMSNorm that follows a product which adds to the residual stream, where the product's last launch has whole
// rows in hand (the launch that adds the shares of K): weight null for none.
struct ThenNorm {
  const float* weight;   // [N]
  float eps;
  bf16_t* out;           // [M, ld]: rmsnorm(residual's new rows) * weight
  int64_t ld;
};
constexpr ThenNorm kNoNorm = {nullptr, 0.f, nullptr, 0};

// The shares added to the residual stream as in split_sum_kernel, by a block per row that keeps the row in registers
// (K4 groups of four columns a thread) and goes on to normalise it: the sums, the threads' places and the arithmetic
// are those of split_sum_kernel followed by rmsnorm_kernel (elementwise.hip), value for value, without the second
// launch and its trip through memory. Everything a thread reads for up to four of its groups is asked for at once
// (every thread issues every load, from the row's last group where its own lies past the end, and from the last
// share where there are fewer than eight): the shares come from memory, and a thread that took its groups one
// after the other would wait a memory latency for each (7B sizes, 64 rows of 3,584: the loop cost more than the
// norm's own launch saves).
template <int K4>
__global__ void __launch_bounds__(256) split_sum_norm_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ parts, int shares,
                                                             int M, int N, ThenNorm then) {
  __shared__ float scratch[4];
  constexpr int kTogether = K4 < 4 ? K4 : 4;
  const int m = blockIdx.x, groups = N / 4;
  const int64_t part = static_cast<int64_t>(M) * N;
  float4 xs[K4], ws[K4];
#pragma unroll
  for (int i0 = 0; i0 < K4; i0 += kTogether) {
    float4 old[kTogether], v[kTogether][8];
#pragma unroll
    for (int j = 0; j < kTogether; ++j) {
      const int g = threadIdx.x + 256 * (i0 + j), gc = g < groups ? g : groups - 1;
      const float* src = parts + static_cast<int64_t>(m) * N + 4 * gc;
      old[j] = *reinterpret_cast<const float4*>(out + static_cast<int64_t>(m) * ldo + 4 * gc);
      ws[i0 + j] = reinterpret_cast<const float4*>(then.weight)[gc];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[j][u] = *reinterpret_cast<const float4*>(src + min(u, shares - 1) * part);
    }
#pragma unroll
    for (int j = 0; j < kTogether; ++j) {
      const int g = threadIdx.x + 256 * (i0 + j), gc = g < groups ? g : groups - 1;
      float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (u < shares) { sum.x += v[j][u].x; sum.y += v[j][u].y; sum.z += v[j][u].z; sum.w += v[j][u].w; }
      for (int s0 = 8; s0 < shares; s0 += 8) {     // (more than eight shares: the next eight, together again)
        const float* src = parts + static_cast<int64_t>(m) * N + 4 * gc;
        float4 more[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) more[u] = *reinterpret_cast<const float4*>(src + min(s0 + u, shares - 1) * part);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < shares) { sum.x += more[u].x; sum.y += more[u].y; sum.z += more[u].z; sum.w += more[u].w; }
      }
      const bool mine = g < groups;
      xs[i0 + j] = mine ? make_float4(old[j].x + sum.x, old[j].y + sum.y, old[j].z + sum.z, old[j].w + sum.w) : make_float4(0.f, 0.f, 0.f, 0.f);
      if (!mine) ws[i0 + j] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (mine) *reinterpret_cast<float4*>(out + static_cast<int64_t>(m) * ldo + 4 * g) = xs[i0 + j];
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < K4; ++i) {      // ascending columns within the thread
    ss += xs[i].x * xs[i].x;
    ss += xs[i].y * xs[i].y;
    ss += xs[i].z * xs[i].z;
    ss += xs[i].w * xs[i].w;
  }
  ss = block_sum<float, 256>(ss, scratch);
  const float scale = 1.f / sqrtf(ss / static_cast<float>(N) + then.eps);
#pragma unroll
  for (int i = 0; i < K4; ++i) {
    const int g = threadIdx.x + 256 * i;
    if (g < groups)
      *reinterpret_cast<uint2*>(then.out + static_cast<int64_t>(m) * then.ld + 4 * g) =
          make_uint2(pack_bf16x2(xs[i].x * scale * ws[i].x, xs[i].y * scale * ws[i].y), pack_bf16x2(xs[i].z * scale * ws[i].z, xs[i].w * scale * ws[i].w));
  }
}

// K shared out among the blocks of a launch (tiles of 64 rows x 64 WTN columns, a ring of S slabs), and a second
// launch that adds the shares and runs the epilogue. The parts lie in the workspace as [shares, M, N] floats.
template <int kEpilogue, typename TO, int WTN, int S, int WTM = 1>
static int launch_dma_sliced(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, int64_t ldw, const float* bias, int M, int N, int K,
                             int shares, hipStream_t stream, const ThenNorm& then, int* then_done) {
  const int tiles_n = (N + 64 * WTN - 1) / (64 * WTN), tiles_m = (M + 64 * WTM - 1) / (64 * WTM);
  const Workspace& g_ws = workspace();
  ALOFA_REQUIRE(g_ws.tiles != nullptr && N % 4 == 0 && static_cast<int64_t>(shares) * M * N <= g_ws.tile_floats,
                "gemm_mfma: %d shares of %d x %d sums do not fit the workspace (or N is no multiple of four)", shares, M, N);
  gemm_dma_kernel<kMfStore, float, WTM, WTN, S, 2><<<tiles_n * tiles_m * shares, 256, 0, stream>>>(
      g_ws.tiles, N, static_cast<const bf16_t*>(A), lda, static_cast<const bf16_t*>(W), nullptr, ldw, nullptr, M, N, K, tiles_m, tiles_n, 1, shares);
  if constexpr (kEpilogue == kMfResidual && sizeof(TO) == 4) {
    // the norm behind the product rides on the launch that adds the shares (rows up to 8,192 wide stay in registers)
    if (then.weight != nullptr && N <= 8192 && ldo % 4 == 0 && then.ld % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(then.weight) % 16 == 0 && reinterpret_cast<uintptr_t>(then.out) % 8 == 0) {
      float* o = static_cast<float*>(out);
      if (N <= 1024) split_sum_norm_kernel<1><<<M, 256, 0, stream>>>(o, ldo, g_ws.tiles, shares, M, N, then);
      else if (N <= 2048) split_sum_norm_kernel<2><<<M, 256, 0, stream>>>(o, ldo, g_ws.tiles, shares, M, N, then);
      else if (N <= 4096) split_sum_norm_kernel<4><<<M, 256, 0, stream>>>(o, ldo, g_ws.tiles, shares, M, N, then);
      else split_sum_norm_kernel<8><<<M, 256, 0, stream>>>(o, ldo, g_ws.tiles, shares, M, N, then);
      *then_done = 1;
      return 0;
    }
  }
  const int64_t threads = static_cast<int64_t>(M) * (N / 4);
  split_sum_kernel<kEpilogue, TO><<<static_cast<int>((threads + 255) / 256), 256, 0, stream>>>(static_cast<TO*>(out), ldo, g_ws.tiles, shares, bias, M, N);
  return 0;
}

template <int kEpilogue, typename TO, int WTM, int WTN, int S>
static int launch_dma(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, int64_t ldw, const float* bias, int M, int N, int K,
                      hipStream_t stream, const void* W2 = nullptr, int own = 0) {
  constexpr int kOutCols = (kEpilogue == kMfSwiglu) ? 32 * WTN : 64 * WTN;     // (gate and up rows of the same columns share a slab)
  const int owned = (own > 0 && own < kOutCols) ? own : kOutCols;
  const int tiles_n = (N + owned - 1) / owned, tiles_m = (M + 64 * WTM - 1) / (64 * WTM);
  // (tiles dealt out die by die at every size: with weights that come from memory it is 3 to 9 % faster here than row
  // by row also where the operands would fit the L2s: 12.4 against 13.3 us for N = 1,152, K = 896 at 2,048 rows)
  const int by_die = 1;
  gemm_dma_kernel<kEpilogue, TO, WTM, WTN, S><<<tiles_n * tiles_m, 256, 0, stream>>>(
      static_cast<TO*>(out), ldo, static_cast<const bf16_t*>(A), lda, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2), ldw, bias, M, N, K,
      tiles_m, tiles_n, by_die, 1, nullptr, nullptr, owned == kOutCols ? 0 : owned);
  return 0;
}

// Whether `tiles` blocks that run one per compute unit come out in nearly full rounds of the chip (the last
// round at least seven eighths full on average over the rounds).
static bool fills_rounds(int64_t tiles) {
  const int64_t rounds = (tiles + 255) / 256;
  return tiles * 8 >= rounds * 256 * 7;
}

// How many shares of K make `tiles` output tiles (of tile_floats each) fill the chip: doubled while the blocks
// stay within two per compute unit, every share keeps at least four slabs and the partial tiles fit the workspace.
static int k_shares(int64_t tiles, int64_t tile_floats, int K) {
  const Workspace& g_ws = workspace();
  if (g_ws.tiles == nullptr || tiles > kGemmCounters) return 1;
  const int slabs = (K + TK - 1) / TK;
  int shares = 1;
  while (shares < 16 && tiles * shares * 2 <= 512 && slabs / (shares * 2) >= 4 && tiles * shares * 2 * tile_floats <= g_ws.tile_floats)
    shares *= 2;
  return shares;
}

// The output columns a block owns where one tile of rows meets gate and up matrices whose whole tiles of 128 columns
// are fewer than the compute units: the columns dealt out evenly over the compute units (at least 16), and the form
// follows from that number (launch_mfma). A compute unit pulls its block's weight rows at a rate of its own, well below
// its share of the memory's, so compute units without a block are lost: gate and up of 18,944 columns in 256 blocks
// of 74 (of tiles that hold 128) 55-58 us at 8 to 64 rows where 148 blocks of 128 or 296 of 64 take 62-69; of 8,960
// columns 15.2-16.1 against 17.3-20.0; of 13,824 57-61 against 60-66; of 11,008 24.0-25.2 against 25.4-26.3; no
// difference at 27,648 (216 blocks of 128 already read at the memory's rate) and 4,864 (the launch itself). 0: whole
// tiles.
static int owned_columns(int N) {
  const int units = compute_units();
  if ((N + 127) / 128 >= units) return 0;
  const int own = (N + units - 1) / units;
  return own < 16 ? 16 : own;
}

template <int kEpilogue, typename TO>
static int launch_mfma(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                       const float* bias, int M, int N, int K, hipStream_t stream, const ThenNorm& then, int* then_done) {
  if constexpr (kEpilogue != kMfArgmax) {
    if (wide_pays<kEpilogue>(M, N, K)) {
      if (launch_wide<kEpilogue, TO, 256, 256, 4, 2, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2)) return 1;
      return check_launch("gemm_wide");
    }
  }
  if constexpr (kEpilogue == kMfSwiglu) {
    // A block computes gate and up of the same 64 columns. With K a multiple of 64 and tiles that do not fill the
    // chip twice over, the slabs go straight from memory into a ring in LDS (0.5B sizes, us against the kernel
    // that brings them in through registers with 128-row tiles, one slab ahead):
    //  * up to 64 rows, and further while the tiles of 64 rows are no more than the compute units: such tiles
    //    (64 gate + 64 up columns; 128 + 128 for a long and wide pair of matrices, see below),
    //    a ring of four where K is short (one block per compute unit), of three otherwise (9.9, 10.6, 11.4, 11.4
    //    at 17, 32, 64, 192 rows against 11.8, 12.2, 12.3 through registers and 22.4; 7B sizes at 64 rows: 70.8
    //    against 72.5);
    //  * then, while the tiles of 128 rows are no more than the compute units: those, a ring of three (14.5 at
    //    256 rows, 14.8 at 384 against 22.6 and 22.8);
    //  * up to two such tiles per compute unit: a ring of two, two blocks per compute unit (22.5 at 512 rows,
    //    23.6 at 768 against 24.1 and 25.4);
    //  * more tiles: through registers (30.8 at 1,024 rows against 39.9).
    const int64_t col_tiles = (N + 63) / 64;
    const int64_t tiles_64 = col_tiles * ((M + 63) / 64), tiles_128 = col_tiles * ((M + 127) / 128);
    const bool ring = K % TK == 0;
    const int own = M <= 64 ? owned_columns(N) : 0;     // (one tile of rows: what a block owns if the blocks are dealt out evenly, 0 if whole tiles fill the chip)
    if (ring && own > 0 && K >= 2048) {
      if (own <= 64) {
        if (launch_dma<kEpilogue, TO, 1, 2, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, own)) return 1;
      } else {
        if (launch_dma<kEpilogue, TO, 1, 4, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, own)) return 1;
      }
    } else if (ring && own > 0 && own <= 64) {
      if (own <= 32) {
        if (launch_dma<kEpilogue, TO, 1, 1, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, own)) return 1;
      } else {
        if (launch_dma<kEpilogue, TO, 1, 2, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, own)) return 1;
      }
    } else
    if (ring && (M <= 64 || tiles_64 <= 256)) {
      if (K >= 2048 && ((N + 127) / 128 >= 192 || ((N + 127) / 128 >= 128 && M > 32))) {
        // a long and wide pair of matrices: 128 gate + 128 up columns per block, a ring of three, one block per
        // compute unit; the rows are read half as often (32B sizes: 105, 107, 109 us at 16, 32, 64 rows against
        // 114, 120, 125; with fewer such tiles than three quarters of the compute units only from 33 rows on: 7B
        // sizes, 148 tiles, 64.1 against 62.4 at 16 rows, 67.6 against 70.7 at 64)
        if (launch_dma<kEpilogue, TO, 1, 4, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, 0)) return 1;
      } else if (K < 2048) {
        // (up to 64 rows and fewer tiles than half the compute units: tiles of 32 outputs, whose gate and up halves
        // are computed by different waves and meet in LDS; N = 4,864, K = 896 at 17 to 64 rows 8.5-9.4 us against
        // 9.9-11.2)
        if (M <= 64 && (N + 63) / 64 < 128) {
          if (launch_dma<kEpilogue, TO, 1, 1, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, 0)) return 1;
        } else
        if (launch_dma<kEpilogue, TO, 1, 2, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, 0)) return 1;
      } else {
        if (launch_dma<kEpilogue, TO, 1, 2, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2, 0)) return 1;
      }
    } else if (ring && tiles_128 <= 256) {
      if (launch_dma<kEpilogue, TO, 2, 2, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2)) return 1;
    } else if (ring && tiles_128 < 512) {
      if (launch_dma<kEpilogue, TO, 2, 2, 2>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2)) return 1;
    } else if (ring && K >= 2048 && fills_rounds(static_cast<int64_t>((N + 127) / 128) * ((M + 127) / 128))) {
      // many rows against a long and wide pair of matrices: tiles of 128 rows x (128 gate + 128 up) columns, a ring of
      // three, one block per compute unit, where such tiles come out in nearly full rounds of the chip (2,048 rows,
      // 7B sizes: 705 against 738 us; 32B sizes: 1,322 against 1,418; with a short K the tiles below stay ahead:
      // 0.5B sizes 65.8 against 60.1)
      if (launch_dma<kEpilogue, TO, 2, 4, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream, W2)) return 1;
    } else if (M > 64 && tiles_128 >= 256) {
      // (a tile of 128 x 128 outputs, 256 rows of W, leaves room for one block per compute unit only: slower)
      if (launch_tile<kEpilogue, TO, 2, 2, 1, false>((N + 63) / 64, (M + 127) / 128, 1, out, ldo, A, lda, W, W2, ldw, bias, M, N, K, stream)) return 1;
    } else {
      if (launch_tile<kEpilogue, TO, 1, 2, 2, false>((N + 63) / 64, (M + 63) / 64, 1, out, ldo, A, lda, W, W2, ldw, bias, M, N, K, stream)) return 1;
    }
    return check_launch("gemm_mfma");
  } else {
    // Big tiles (one slab ahead) when they fill the chip: about two blocks per compute unit, which hide one
    // another's waits. Small tiles (two slabs ahead) otherwise: few big tiles, each alone on its compute
    // unit, were slower here even with four slabs ahead. Where even the small tiles are too few, K is
    // shared out among blocks as well.
    const int64_t big_blocks = static_cast<int64_t>((N + 127) / 128) * ((M + 127) / 128);
    const int64_t tiles_192 = static_cast<int64_t>((N + 191) / 192) * ((M + 127) / 128);
    const int64_t tiles_256 = static_cast<int64_t>((N + 255) / 256) * ((M + 127) / 128);
    const int64_t rounds_192 = (tiles_192 + 255) / 256, rounds_256 = (tiles_256 + 255) / 256;
    if (M > 64 && K % TK == 0 && K >= 2048 && rounds_192 * 192 < rounds_256 * 256 &&
        (rounds_192 == 1 ? tiles_192 >= 128 : tiles_192 * 16 >= rounds_192 * 256 * 13)) {
      // tiles of 128 x 192, a ring of three, one block per compute unit, where their rounds of the chip cover
      // fewer columns than those of the 256-wide tiles below and are full enough: a single round on half of the
      // compute units or more (1,024 rows: 235 against 307 us for N = 3,584, K = 18,944, 390 against 500 for
      // N = 5,120, K = 27,648, 61 against 75 for N = 4,608, K = 3,584), or several at least 13/16 full (2,048 rows:
      // 762 against 825 for N = 5,120, K = 27,648; 4,096 rows: 189 against 203 for N = 4,608, K = 3,584)
      if (launch_dma<kEpilogue, TO, 2, 3, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream)) return 1;
    } else
    if (M > 64 && K % TK == 0 && K >= 2048 && big_blocks >= 256 && fills_rounds(tiles_256)) {
      // tiles of 128 x 256, a ring of three, one block per compute unit, where such tiles come out in nearly full
      // rounds of the chip (2,048 rows: 343 against 368 us for N = 3,584, K = 18,944, 198 against 234 for N = 7,168,
      // K = 5,120; where the last round is half empty they lose: 138 against 121 for N = 4,608, K = 3,584)
      if (launch_dma<kEpilogue, TO, 2, 4, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream)) return 1;
    } else
    if (M <= 64 && (N + 127) / 128 >= 256) {
      // one tile of rows against a long matrix (the vocabulary): tiles of 64 rows, so that no empty rows are staged
      if (launch_tile<kEpilogue, TO, 1, 2, 2, false>((N + 127) / 128, 1, 1, out, ldo, A, lda, W, W2, ldw, bias, M, N, K, stream)) return 1;
    } else if (big_blocks >= 512) {
      if (launch_tile<kEpilogue, TO, 2, 2, 1, false>((N + 127) / 128, (M + 127) / 128, 1, out, ldo, A, lda, W, W2, ldw, bias, M, N, K, stream)) return 1;
    } else if (big_blocks >= 256 && K % TK == 0) {
      // One to two big tiles per compute unit: a ring of two slabs filled straight from memory, two blocks per
      // compute unit, all of them resident at once. (2,048 rows, weights from memory, against the small tiles
      // below: 71 against 102 us for 3,584 x 3,584, 335 against 513 for N = 3,584, K = 18,944. With more tiles
      // than two per compute unit the three resident blocks of the kernel above do better: 107 against 137 us
      // for N = 4,608, K = 3,584.)
      if (launch_dma<kEpilogue, TO, 2, 2, 2>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream)) return 1;
    } else {
      const int tiles_n = (N + 63) / 64, tiles_m = (M + 63) / 64;
      const bool ring = K % TK == 0, long_k = K >= 32 * TK;
      const int64_t tiles_128x64 = static_cast<int64_t>((M + 127) / 128) * tiles_n;
      // With a short K a share of it is too short to pay for the hand-over: small tiles unshared, slabs straight
      // from memory (0.5B sizes, 96 to 768 rows: 8.1-8.5 us against 8.8-10.8 for N = 1,152, K = 896).
      const int shares = (ring && !long_k) ? 1 : k_shares(static_cast<int64_t>(tiles_n) * tiles_m, 64 * 64, K);
      // Up to 64 rows against a matrix of few columns and a long K: with few column tiles the blocks that arrive
      // last, one per tile, would add all the shares of their tiles while the rest of the chip is done. Tiles of
      // 128 columns instead, K in as many shares as fill the chip once (four slabs each at least), every block
      // leaving its sums as they are, and a second launch of a thread per four outputs that adds the shares in
      // their order (us against the hand-over, 64 rows: N = 4,608, K = 3,584 14.2 against 18.7; 3,584 x 3,584
      // 13.6 against 16.5; N = 3,584, K = 18,944 35.0 against 40.6; N = 1,536, K = 8,960 16.4 against 21.3; with
      // 40 column tiles and more the hand-over is ahead: N = 5,120, K = 5,120 at 32 rows 25.3 against 23.1,
      // N = 7,168 29.3 against 24.1).
      // More than 64 rows, a long K and too few tiles of 128 x 128 for the chip (a down projection in a prefill of
      // a small model, a portion of a prompt against the projections of a large one): such tiles with K in two to
      // eight shares, as many as fill the chip once, and the second launch that adds them (us against the rules
      // below: N = 896, K = 4,864 at 2,048 rows 32.0 against 33.7, at 1,024 rows 21.8 against 28.7; N = 3,584,
      // K = 18,944 at 128, 256, 384 rows 43.6, 61.1, 76.8 against 55.4, 89.7, 120.7; N = 5,120, K = 27,648 at 128
      // and 256 rows 74 and 110 against 135 and 178; 5,120 x 5,120 at 256 rows 32.1 against 42.9; 3,584 x 3,584 at 384 rows 23.9 against 30.0; with K = 2,048 it loses,
      // N = 2,560 at 512 rows 20.0 against 16.9).
      const int64_t tiles_128x128 = static_cast<int64_t>((M + 127) / 128) * ((N + 127) / 128);
      int tall_shares = static_cast<int>(256 / tiles_128x128);      // as many as fill the chip once: up to eight, of sixteen slabs or more
      if (tall_shares > 8) tall_shares = 8;
      if (tall_shares > K / TK / 16) tall_shares = K / TK / 16;
      if (tiles_128x128 * tall_shares < 160) tall_shares = 0;       // (too few blocks for the chip: the rules below)
      const bool tall = tall_shares > 1 && K >= 3072 && M > 64;
      // (the tiles of 64 x 128 also up to 256 rows, for K from 3,072, where those of 128 x 128 are too few even in
      // shares: N = 896, K = 4,864 at 65, 128 and 256 rows 10.4, 12.3 and 14.0 us against 15.0, 15.1 and 16.8;
      // N = 2,048, K = 11,008 at 128 rows 22.2 against 24.8)
      const int wide_tiles = ((N + 127) / 128) * tiles_m, all_slabs = K / TK;
      const int per_share = max(4, (all_slabs * wide_tiles + 255) / 256), slices = (all_slabs + per_share - 1) / per_share;
      if (kEpilogue != kMfSwiglu && ring && long_k && (M <= 64 || (M <= 256 && !tall && K >= 3072)) && wide_tiles <= 36 && N % 4 == 0 && slices > 1 &&
          static_cast<int64_t>(slices) * M * N <= workspace().tile_floats) {
        if constexpr (kEpilogue != kMfSwiglu) {
          if (launch_dma_sliced<kEpilogue, TO, 2, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, slices, stream, then, then_done)) return 1;
        }
      } else
      if (tall && kEpilogue != kMfSwiglu && ring && N % 4 == 0 &&
          static_cast<int64_t>(tall_shares) * M * N <= workspace().tile_floats) {
        if constexpr (kEpilogue != kMfSwiglu) {
          if (launch_dma_sliced<kEpilogue, TO, 2, 3, 2>(out, ldo, A, lda, W, ldw, bias, M, N, K, tall_shares, stream, then, then_done)) return 1;
        }
      } else
      if (ring && long_k && tiles_128x64 >= 144 && tiles_128x64 <= 256) {
        // Tiles of 128 x 64 that fill most of the chip once, and a long K: one block per compute unit with a ring
        // of four (35.8 against 38.8 us for N = 896, K = 4,864 at 2,048 rows; 28.8 against 36.1 with K shared out
        // for N = 4,608, K = 3,584 at 256 rows, 121 against 151 for N = 3,584, K = 18,944 at 384 rows; fewer tiles
        // do better with K shared out, 26.1 against 30.3 for 3,584 x 3,584 at 256 rows; with a short K, or with
        // more tiles than compute units, the small tiles below do better: 11.6 against 10.4 us for 896 x 896)
        if (launch_dma<kEpilogue, TO, 2, 1, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream)) return 1;
      } else if (shares > 1) {
        // K shared out among blocks: with weights of 32 MB or more the slabs go straight into a ring of three in
        // LDS here too (N = 5,120, K = 27,648 at 32 rows: 75 against 85 us; N = 3,584, K = 18,944 at 16 rows: 34.4
        // against 36.1; N = 4,608, K = 3,584 at 16 rows: 14.6 against 16.2); smaller ones gain nothing by it
        // (3,584 x 3,584 at 16 rows: 15.7 against 15.4; N = 896, K = 4,864 at 96 rows: 19.5 against 18.2)
        if (ring && static_cast<int64_t>(N) * K * 2 >= (32ll << 20)) {
          if (launch_dma_shared<kEpilogue, TO, 1, 1, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, shares, stream)) return 1;
        } else
        if (launch_tile<kEpilogue, TO, 1, 1, 2, true>(tiles_n, tiles_m, shares, out, ldo, A, lda, W, W2, ldw, bias, M, N, K, stream)) return 1;
      } else if (ring) {
        // small tiles, slabs straight from memory into a ring of three (against the kernel below, same conditions:
        // 13.3 against 15.8 us for N = 1,152, K = 896; 10.4 against 12.2 for 896 x 896; 38.8 against 44.6 for
        // N = 896, K = 4,864; a ring of two is slower than either when the weights come from memory: 60 us)
        if (launch_dma<kEpilogue, TO, 1, 1, 3>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream)) return 1;
      } else {
        if (launch_tile<kEpilogue, TO, 1, 1, 2, false>(tiles_n, tiles_m, 1, out, ldo, A, lda, W, W2, ldw, bias, M, N, K, stream)) return 1;
      }
    }
    return check_launch("gemm_mfma");
  }
}

}  // namespace alofa

using namespace alofa;

// bfloat16 A [M, K] and W [N, K] (W2 for the swiglu epilogue); K a multiple of 8, rows 16-byte
// aligned. Epilogues: 0 store (+ bias) as o_dtype, 1 add to the float residual, 2 swiglu.
// then_w (may be null; residual epilogue only): an RMSNorm (then_w [N], then_eps) of the residual's new rows is
// wanted in then_out (bfloat16 [M, then_ld]) afterwards. Where the product's last launch has whole rows in hand it
// writes them and sets *then_done to 1; otherwise *then_done stays 0 and the norm is the caller's to run.
extern "C" int alofa_gemm_mfma(void* out, int o_dtype, int64_t ldo, const void* A, int64_t lda, const void* W,
                               const void* W2, int64_t ldw, const float* bias, int M, int N, int K, int epilogue,
                               const float* then_w, float then_eps, void* then_out, int64_t then_ld, int* then_done,
                               hipStream_t stream) {
  ALOFA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_mfma: M=%d N=%d K=%d must be positive", M, N, K);
  ALOFA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_mfma: K=%d, lda=%lld, ldw=%lld must be multiples of 8", K,
                static_cast<long long>(lda), static_cast<long long>(ldw));
  ALOFA_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(W2) % 16 == 0, "gemm_mfma: operands must be 16-byte aligned");
  ALOFA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_mfma: a leading dimension is shorter than its row");
  ALOFA_REQUIRE(then_w == nullptr || (epilogue == kMfResidual && then_out != nullptr && then_ld >= N && then_eps > 0.f && then_done != nullptr),
                "gemm_mfma: a norm behind the product goes with the residual epilogue, an output of the product's shape and a positive eps");
  const ThenNorm then{then_w, then_eps, static_cast<bf16_t*>(then_out), then_ld};
  int none = 0;
  int* done = then_done ? then_done : &none;
  *done = 0;
  if (epilogue == kMfStore && o_dtype == kBF16)
    return launch_mfma<kMfStore, bf16_t>(out, ldo, A, lda, W, nullptr, ldw, bias, M, N, K, stream, kNoNorm, done);
  if (epilogue == kMfStore && o_dtype == kF32)
    return launch_mfma<kMfStore, float>(out, ldo, A, lda, W, nullptr, ldw, bias, M, N, K, stream, kNoNorm, done);
  if (epilogue == kMfResidual && o_dtype == kF32)
    return launch_mfma<kMfResidual, float>(out, ldo, A, lda, W, nullptr, ldw, nullptr, M, N, K, stream, then, done);
  if (epilogue == kMfSwiglu && o_dtype == kBF16) {
    ALOFA_REQUIRE(W2 != nullptr, "gemm_mfma: the swiglu epilogue needs the up matrix");
    return launch_mfma<kMfSwiglu, bf16_t>(out, ldo, A, lda, W, W2, ldw, nullptr, M, N, K, stream, kNoNorm, done);
  }
  ALOFA_REQUIRE(false, "gemm_mfma: unsupported epilogue %d with out dtype %d", epilogue, o_dtype);
}

// The same product by the tiles of 256 x 256 with eight waves whatever the sizes (alofa_gemm_mfma takes them where they
// pay): K a multiple of 32. The operands as for alofa_gemm_mfma; norm_w and eps stand where alofa_gemm_skinny has them
// and must be null and zero (no norm rides on this kernel).
extern "C" int alofa_gemm_wide(void* out, int o_dtype, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                               const float* bias, int M, int N, int K, int epilogue, const float* norm_w, float eps, hipStream_t stream) {
  ALOFA_REQUIRE(M > 0 && N > 0 && K > 0 && K % 32 == 0, "gemm_wide: M=%d N=%d K=%d must be positive, K a multiple of 32", M, N, K);
  ALOFA_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldo >= N, "gemm_wide: lda=%lld, ldw=%lld must be multiples of 8 and cover K, ldo=%lld cover N",
                static_cast<long long>(lda), static_cast<long long>(ldw), static_cast<long long>(ldo));
  ALOFA_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 && reinterpret_cast<uintptr_t>(W2) % 16 == 0,
                "gemm_wide: operands must be 16-byte aligned");
  ALOFA_REQUIRE(norm_w == nullptr && eps == 0.f, "gemm_wide: no norm rides on this kernel");
  int failed = 1;
  if (epilogue == kMfStore && o_dtype == kBF16) failed = launch_wide<kMfStore, bf16_t, 256, 256, 4, 2, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream);
  else if (epilogue == kMfStore && o_dtype == kF32) failed = launch_wide<kMfStore, float, 256, 256, 4, 2, 4>(out, ldo, A, lda, W, ldw, bias, M, N, K, stream);
  else if (epilogue == kMfResidual && o_dtype == kF32) failed = launch_wide<kMfResidual, float, 256, 256, 4, 2, 4>(out, ldo, A, lda, W, ldw, nullptr, M, N, K, stream);
  else if (epilogue == kMfSwiglu && o_dtype == kBF16 && W2 != nullptr) failed = launch_wide<kMfSwiglu, bf16_t, 256, 256, 4, 2, 4>(out, ldo, A, lda, W, ldw, nullptr, M, N, K, stream, W2);
  else ALOFA_REQUIRE(false, "gemm_wide: unsupported epilogue %d with out dtype %d", epilogue, o_dtype);
  if (failed) return 1;
  return check_launch("gemm_wide");
}

// out[m] = the column n with the highest sum_k A[m, k] * W[n, k] (the lowest n among equals), for M <= 64 rows
// against a long matrix: the product's blocks leave candidates instead of the M x N outputs (scratch: at least
// 4 * M * ceil(N / 128) floats), a second kernel takes the best of them; store and store_index as for
// alofa_argmax_to_store (both null: no store).
extern "C" int alofa_gemm_argmax(int32_t* out, int32_t* store, const int32_t* store_index, float* scratch, int64_t scratch_floats,
                                 const void* A, int64_t lda, const void* W, int64_t ldw, int M, int N, int K, hipStream_t stream) {
  ALOFA_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_argmax: M=%d (1..64) N=%d K=%d", M, N, K);
  ALOFA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K, "gemm_argmax: K=%d, lda=%lld, ldw=%lld must be multiples of 8 and cover K", K,
                static_cast<long long>(lda), static_cast<long long>(ldw));
  ALOFA_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0, "gemm_argmax: operands must be 16-byte aligned");
  const int tiles_n = (N + 127) / 128, parts = 2 * tiles_n;
  ALOFA_REQUIRE(out != nullptr && scratch != nullptr && scratch_floats >= 2ll * M * parts, "gemm_argmax: the scratch holds %lld floats, %lld are needed",
                static_cast<long long>(scratch_floats), 2ll * M * parts);
  if (launch_tile<kMfArgmax, float, 1, 2, 2, false>(tiles_n, 1, 1, scratch, parts, A, lda, W, nullptr, ldw, nullptr, M, N, K, stream)) return 1;
  if (check_launch("gemm_argmax")) return 1;
  return alofa_argmax_parts(out, store, store_index, scratch, reinterpret_cast<const int32_t*>(scratch + static_cast<int64_t>(M) * parts), M, parts, N, stream);
}
