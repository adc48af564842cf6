// Paged causal grouped-query attention for prompt portions, bfloat16 on MFMA,
// with a running softmax so that no score matrix is ever stored.
//
// A block serves, with TEAMS teams of WPT wavefronts each, either (kShare false)
// 64 consecutive query rows of one request and one query head, every wave of a
// team owning 16 rows (WPT = 4); or (kShare true) 16 consecutive query rows and
// up to WPT query heads of one key head, every wave of a team owning one head:
// the heads of a group read the same keys and values, so a tile that is fetched
// and staged once serves all of them (a fetch and a staging per head cost about
// as much as the head's arithmetic).
// The visible keys are walked in tiles of 64 that start at absolute multiples
// of 64; the teams take the tiles in turn (a row's chain of dependent tiles is
// TEAMS times shorter, and the teams' waves fill one another's stalls) and
// their running states meet in LDS at the end, combined in team order. Per
// tile a team stages the keys [64, d] and the values transposed [d, 64] in LDS.
//
// Both products are taken transposed, so that one lane's data stays with one
// query row throughout (v_mfma_f32_16x16x32_bf16; lane l: A row and B column
// l % 16, D column l % 16 and rows 4 * (l / 16) .. + 3):
//   S^T[key, q] = K[key, :] . Q[q, :]      A = keys from LDS, B = queries (registers)
//   O^T[c, q] += V^T[c, key] * P^T[key, q]  A = values^T from LDS, B = weights (registers)
// After the first product of a 32-key half lane l holds, for query l % 16, the
// scores of keys 4 g + r and 16 + 4 g + r (g = l / 16, r = 0..3); these eight are
// exactly the reduction slots of the second product when the values are read in
// the same order, so the weights never leave their registers.
// Scores, the running maximum, the weights and their sum are float; the
// weights are rounded to bfloat16 only as MFMA operands.
// With RW = 32 a wave owns 32 query rows instead of 16 (v_mfma_f32_32x32x16_bf16; lane l: A row and B column
// l % 32, reduction slots 8 (l / 32) .. + 7, D column l % 32 and rows 8 j + 4 (l / 32) + r for j, r = 0..3): a
// fragment of keys or values read from LDS then feeds twice the arithmetic, and LDS reads are what the
// 16-row form waits for. After the first product of a 32-key half lane l holds, for query l % 32, the scores
// of keys 8 j + 4 h + r (h = l / 32); those of j = 0, 1 are the eight reduction slots of one second product
// and those of j = 2, 3 of the next, with the values read in the same order.
// Cache layout: keys [block, kv_head, slot_in_block, d], values transposed [block, kv_head, d, slot_in_block]:
// eight consecutive keys of a channel are one 16-byte load, staged as they are.
#include "common.h"

#include <float.h>

namespace alofa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// the larger / the sum of v in lanes l and l ^ 32
__device__ __forceinline__ float halves_max(float v) {
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float halves_sum(float v) {
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

constexpr int BQ = 64;    // query rows per block
constexpr int KPAD = 8, VPAD = 8;

// tiles: int32 [n_blocks, 2, 4]: a block serves up to two runs of rows, one after the other, each
// (request index, first row in the packed batch, rows (<= 64; 0: none), position of the first row). The caller
// pairs long runs with short ones so that blocks carry about the same number of key tiles.
// kShare: blockIdx.y = key head * chunks + chunk of up to WPT query heads of its group; blockIdx.z = which RW rows of the run.
template <int DT, int TEAMS, int WPT, bool kShare, int RW = 16, int KT = 64>  // DT = d / 16; RW: query rows per wave (16 or 32); KT: keys per tile (64; 32 with RW = 32)
__global__ void __launch_bounds__(64 * WPT * TEAMS, (RW == 32 && 64 * WPT * TEAMS <= 256) ? 2 : 1) attention_prefill_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_table,
    int max_blocks, const int32_t* __restrict__ tiles, int heads, int kv_heads, int bs_shift, int window,
    float scale) {
  constexpr int d = DT * 16;
  constexpr int BKV = KT;
  static_assert(KT == 64 || (KT == 32 && RW == 32), "tiles of 64 keys, or of 32 with 32 rows a wave");
  constexpr int DS = RW == 32 ? DT : (d + 31) / 32;   // steps of 32 (RW = 32: of 16) along d in the first product
  constexpr int OT = RW == 32 ? (d + 31) / 32 : DT;   // output tiles of 16 (RW = 32: of 32) channels
  constexpr int OV = RW == 32 ? 16 : 4;               // ... each this many values per lane
  static_assert(RW == 16 || RW == 32, "a wave owns 16 or 32 query rows");
  constexpr int KROW = d + KPAD, VROW = BKV + VPAD;
  // per team: its key tile and its transposed value tile; at the end the same room takes the team's
  // running state (per lane its maximum, its sum and its 4 * DT channels)
  constexpr int kTeamThreads = 64 * WPT;
  static_assert(kShare || WPT * RW == BQ, "without sharing a team's waves own the 16- or 32-row groups of a run");
  // (RW = 32 reads value rows up to the next multiple of 32 channels; what lies past d is never stored)
  constexpr int kStageBytes = (BKV * KROW + (RW == 32 ? 32 * OT : d) * VROW) * 2, kStateBytes = kTeamThreads * (OV * OT + 2) * 4;
  constexpr int kTeamBytes = (((TEAMS > 1 && kStateBytes > kStageBytes) ? kStateBytes : kStageBytes) + 15) / 16 * 16;   // (one team hands no state over)
  __shared__ __attribute__((aligned(16))) char team_room[TEAMS * kTeamBytes];
  // (the wave's number as a scalar: what depends on it alone, the team's tile and whether it is whole, then stays out of the vector unit)
  const int wave_of_block = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int team = wave_of_block / WPT;
  bf16_t* Ks = reinterpret_cast<bf16_t*>(team_room + team * kTeamBytes);
  bf16_t* Vt = Ks + BKV * KROW;

  const int wave = wave_of_block % WPT, lane = threadIdx.x % 64, tid = wave * 64 + lane;
  const int c16 = lane % 16, g = lane / 16;
  const int r32 = lane % 32, h = lane / 32;
  const int group = heads / kv_heads, chunks = (group + WPT - 1) / WPT;
  // the query head this wave serves (kShare: a wave past the group's end helps with staging only), and its key head
  const int hk = kShare ? blockIdx.y / chunks : blockIdx.y / group;
  const bool head_ok = !kShare || (blockIdx.y % chunks) * WPT + wave < group;
  const int head = kShare ? hk * group + (head_ok ? (blockIdx.y % chunks) * WPT + wave : 0) : blockIdx.y;
  for (int part = 0; part < 2; ++part) {
  const int32_t* tile = tiles + 8 * blockIdx.x + 4 * part;
  // kShare: the block takes rows RW z .. of the run (fewer at the run's end; none: the block has nothing to do in this run)
  const int sub = kShare ? RW * blockIdx.z : 0;
  const int req = tile[0], row0 = tile[1] + sub, pos0 = tile[3] + sub;
  const int n_rows = kShare ? min(tile[2] - sub, RW) : tile[2];
  if (tile[2] <= 0) break;    // uniform over the block
  if (n_rows <= 0) continue;
  __syncthreads();            // the first run's last tile has been read by every wave
  const int32_t* table = block_table + static_cast<int64_t>(req) * max_blocks;

  // this lane's query row and its fragments of Q
  const int my_row = RW == 32 ? (kShare ? r32 : wave * 32 + r32) : (kShare ? c16 : wave * 16 + c16);  // within the block's rows
  const bool row_ok = my_row < n_rows && head_ok;
  const int my_pos = pos0 + my_row;
  bf16x8 qf[DS];
#pragma unroll
  for (int ds = 0; ds < DS; ++ds) {
    uint4 v = make_uint4(0, 0, 0, 0);
    const int c = RW == 32 ? ds * 16 + h * 8 : ds * 32 + g * 8;
    if (row_ok && c < d)
      v = *reinterpret_cast<const uint4*>(q + static_cast<int64_t>(row0 + my_row) * q_stride + static_cast<int64_t>(head) * d + c);
    qf[ds] = __builtin_bit_cast(bf16x8, v);
  }

  typedef float out_tile __attribute__((ext_vector_type(OV)));
  out_tile o[OT];
#pragma unroll
  for (int nt = 0; nt < OT; ++nt)
#pragma unroll
    for (int e = 0; e < OV; ++e) o[nt][e] = 0.f;
  float m = -FLT_MAX, l = 0.f;
  const float scale2 = scale * 1.44269504088896340736f;   // scores in units of log2(e)

  // keys the block needs: from the first key its first row sees to the last row's own position
  const int last_pos = pos0 + n_rows - 1;
  const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int t_begin = first_key / BKV, t_end = last_pos / BKV;     // inclusive

  // staging: 16-byte chunks, 64 * d / 8 of K (eight channels of a key) and as many of V^T (eight keys of a
  // channel; one page: pages hold at least eight tokens). Every lane issues every load, from a visible key
  // in place of one that is not (what such a load brings is cleared at staging): loads that are always
  // issued can stay on their way while the tile before is worked on, a load under a branch is waited for at
  // once. The page numbers of a tile are looked up one tile ahead of its keys and values for the same reason.
  constexpr int kChunks = BKV * d / 8;
  constexpr int kPerThread = (kChunks + kTeamThreads - 1) / kTeamThreads;
  const int page_mask = (1 << bs_shift) - 1;
  const int v_first = first_key & ~7, v_last = last_pos & ~7;    // first and last visible group of eight keys
  uint4 k_reg[kPerThread], v_reg[kPerThread];
  int k_page[kPerThread], v_page[kPerThread];
  auto chunk_of = [&](int j) { const int c = tid + kTeamThreads * j; return c < kChunks ? c : kChunks - 1; };
  auto k_key = [&](int t, int j) { return t * BKV + chunk_of(j) / (d / 8); };
  auto v_key0 = [&](int t, int j) { return t * BKV + (chunk_of(j) % (BKV / 8)) * 8; };
  auto clamp = [](int x, int lo, int hi) { return x < lo ? lo : (x > hi ? hi : x); };
  auto lookup = [&](int t) {
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      k_page[j] = table[clamp(k_key(t, j), first_key, last_pos) >> bs_shift];
      v_page[j] = table[clamp(v_key0(t, j), v_first, v_last) >> bs_shift];
    }
  };
  auto fetch_keys = [&](int t) {
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const int c = chunk_of(j);
      const int key = clamp(k_key(t, j), first_key, last_pos), ch = (c % (d / 8)) * 8;
      k_reg[j] = *reinterpret_cast<const uint4*>(
          k_cache + ((((static_cast<int64_t>(k_page[j]) * kv_heads + hk) << bs_shift) + (key & page_mask)) * d) + ch);
    }
  };
  auto fetch_values = [&](int t) {
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const int c = chunk_of(j);
      const int key0 = clamp(v_key0(t, j), v_first, v_last), channel = c / (BKV / 8);
      v_reg[j] = *reinterpret_cast<const uint4*>(
          v_cache + (((static_cast<int64_t>(v_page[j]) * kv_heads + hk) * d + channel) << bs_shift) + (key0 & page_mask));
    }
  };
  // With 32 rows a wave the next tile's values are asked for only once this tile's scores have become weights:
  // the registers they arrive in are those the scores were in.
  constexpr bool kValuesLate = RW == 32 && DT > 4;
  auto stage = [&](int t) {
    // all 64 keys of the tile visible to the block (all but its first and last tiles): nothing to clear
    const bool whole = t * BKV >= first_key && t * BKV + BKV - 1 <= last_pos;   // uniform over the team
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const int c = tid + kTeamThreads * j;
      if (c < kChunks) {
        uint4 kv = k_reg[j], vv = v_reg[j];
        if (!whole) {
          // what lies beyond the visible keys is not data: it is cleared, so that a weight of zero times it is zero
          const int key = k_key(t, j);
          const uint32_t kk = 0u - static_cast<uint32_t>(key >= first_key && key <= last_pos);   // all ones or zero
          kv = make_uint4(kv.x & kk, kv.y & kk, kv.z & kk, kv.w & kk);
          const int key0 = v_key0(t, j);
          const int lo_e = first_key - key0, hi_e = last_pos - key0 + 1;   // elements lo_e .. hi_e - 1 are visible
          uint32_t w[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const uint32_t keep = 0u - static_cast<uint32_t>(e >= lo_e && e < hi_e);
            w[e / 2] &= (e % 2) ? (keep << 16) | 0x0000ffffu : keep | 0xffff0000u;
          }
          vv = make_uint4(w[0], w[1], w[2], w[3]);
        }
        *reinterpret_cast<uint4*>(&Ks[(c / (d / 8)) * KROW + (c % (d / 8)) * 8]) = kv;
        // row c / 8 of V^T, keys 8 (c % 8) .. + 7 (with tiles of 64 keys). Groups of four keys are permuted within a row by the row's
        // number / 8, so that lanes reading rows r and r + 8 hit different banks: the two groups of this chunk
        // stay in their 16 bytes and change places when that number is odd.
        const int row = c / (BKV / 8), sw = (row >> 3) & 7;
        if (sw & 1) vv = make_uint4(vv.z, vv.w, vv.x, vv.y);
        *reinterpret_cast<uint4*>(&Vt[row * VROW + ((((c % (BKV / 8)) * 2) ^ (sw & 6)) << 2)]) = vv;
      }
    }
  };

  lookup(t_begin + team);
  fetch_keys(t_begin + team);
  fetch_values(t_begin + team);
  lookup(t_begin + team + TEAMS);
  for (int t0 = t_begin; t0 <= t_end; t0 += TEAMS) {     // uniform over the block
    const int t = t0 + team;
    const bool mine = t <= t_end;
    __syncthreads();      // the previous tile has been read by every wave
    if (mine) stage(t);
    __syncthreads();
    if (!mine) continue;
    fetch_keys(t + TEAMS);
    if (!kValuesLate || !head_ok) {
      fetch_values(t + TEAMS);
      lookup(t + 2 * TEAMS);
    }
    if (!head_ok) continue;     // (a wave without a head of its own has done its share of the staging)

    if constexpr (RW == 32) {
    // S^T for the 32-key halves of the tile
    constexpr int KH = BKV / 32;
    f32x16 s[KH];
#pragma unroll
    for (int kh = 0; kh < KH; ++kh) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kh][e] = 0.f;
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        const uint4 kv = *reinterpret_cast<const uint4*>(&Ks[(kh * 32 + r32) * KROW + ds * 16 + h * 8]);
        s[kh] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kv), qf[ds], s[kh], 0, 0, 0);
      }
    }
    // scale, mask, running maximum, as below; element i of this lane: key 32 (i / 16) + 8 ((i % 16) / 4) + 4 h + i % 4 of the tile
    float p[16 * KH];
    float tile_max = -FLT_MAX;
    const bool whole = t * BKV + BKV - 1 <= pos0 && (window <= 0 || t * BKV > last_pos - window);
    float corr, sum = 0.f;
    if (whole) {
#pragma unroll
      for (int i = 0; i < 16 * KH; ++i) tile_max = fmaxf(tile_max, s[i / 16][i % 16]);
      tile_max = halves_max(tile_max);   // over the two lanes that share the query row
      const float m_new = fmaxf(m, tile_max * scale2);
      corr = __builtin_amdgcn_exp2f(m - m_new);
      m = m_new;
#pragma unroll
      for (int i = 0; i < 16 * KH; ++i) {
        p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i / 16][i % 16], scale2, -m_new));
        sum += p[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16 * KH; ++i) {
        const int key = t * BKV + (i / 16) * 32 + ((i % 16) / 4) * 8 + h * 4 + i % 4;
        const bool seen = key <= my_pos && (window <= 0 || key > my_pos - window);
        p[i] = seen ? s[i / 16][i % 16] * scale2 : -FLT_MAX;
        tile_max = fmaxf(tile_max, p[i]);
      }
      tile_max = halves_max(tile_max);
      const float m_new = fmaxf(m, tile_max);
      corr = __builtin_amdgcn_exp2f(m - m_new);
      m = m_new;
#pragma unroll
      for (int i = 0; i < 16 * KH; ++i) {
        p[i] = (p[i] > -FLT_MAX) ? __builtin_amdgcn_exp2f(p[i] - m_new) : 0.f;
        sum += p[i];
      }
    }
    l = l * corr + sum;   // this lane's share of the row's sum; the two lanes of a row meet at the end
    if (kValuesLate) {
      fetch_values(t + TEAMS);
      lookup(t + 2 * TEAMS);
    }
    bf16x8 pf[2 * KH];    // the weights of keys 16 x .. 16 x + 15 of the tile, in this lane's order
#pragma unroll
    for (int x = 0; x < 2 * KH; ++x) {
      const uint4 w = make_uint4(pack_bf16x2(p[8 * x], p[8 * x + 1]), pack_bf16x2(p[8 * x + 2], p[8 * x + 3]),
                                 pack_bf16x2(p[8 * x + 4], p[8 * x + 5]), pack_bf16x2(p[8 * x + 6], p[8 * x + 7]));
      pf[x] = __builtin_bit_cast(bf16x8, w);
    }
    // O^T += V^T P^T, one MFMA per 16 keys: this lane's slots are keys 16 x + 4 h .. + 3 and 16 x + 8 + 4 h .. + 3
    // (leaving the outputs alone where no row's maximum moved, a branch of the wave, is slower: 1.76 against 1.56 ms
    // for 40/8 heads of size 128 and 16k keys)
#pragma unroll
    for (int nt = 0; nt < OT; ++nt) {
      o[nt] *= corr;
      const bf16_t* vrow = &Vt[(nt * 32 + r32) * VROW];
      const int sw = ((nt * 4 + (r32 >> 3)) & 7) << 2;   // this row's permutation of its four-key groups
#pragma unroll
      for (int x = 0; x < 2 * KH; ++x) {
        const uint2 lo = *reinterpret_cast<const uint2*>(vrow + ((x * 16 + h * 4) ^ sw));
        const uint2 hi = *reinterpret_cast<const uint2*>(vrow + ((x * 16 + 8 + h * 4) ^ sw));
        const uint4 vv = make_uint4(lo.x, lo.y, hi.x, hi.y);
        o[nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vv), pf[x], o[nt], 0, 0, 0);
      }
    }
    } else {
    // S^T for the four 16-key quarters of the tile
    f32x4 s[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        const int c = ds * 32 + g * 8;
        uint4 kv = make_uint4(0, 0, 0, 0);
        if (c < d) kv = *reinterpret_cast<const uint4*>(&Ks[(kt * 16 + c16) * KROW + c]);
        s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kv), qf[ds], s[kt], 0, 0, 0);
      }
    }
    // scale, mask, running maximum. Scores are taken in units of log2(e) so that the weights are single
    // exp2 instructions. Tiles that every row of the block sees whole (all but the last one or two) skip
    // the masking: their maximum is taken over the raw scores and the scale goes into the exponent's
    // multiply-add.
    float p[16];
    float tile_max = -FLT_MAX;
    const bool whole = t * BKV + BKV - 1 <= pos0 && (window <= 0 || t * BKV > last_pos - window);
    float corr, sum = 0.f;
    if (whole) {
#pragma unroll
      for (int i = 0; i < 16; ++i) tile_max = fmaxf(tile_max, s[i / 4][i % 4]);
      tile_max = rows_max(tile_max);     // over the four lanes that share the query row
      const float m_new = fmaxf(m, tile_max * scale2);
      corr = __builtin_amdgcn_exp2f(m - m_new);    // 1 while nothing was seen yet (both -FLT_MAX)
      m = m_new;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i / 4][i % 4], scale2, -m_new));
        sum += p[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = t * BKV + (i / 4) * 16 + g * 4 + i % 4;
        const bool seen = key <= my_pos && (window <= 0 || key > my_pos - window);
        p[i] = seen ? s[i / 4][i % 4] * scale2 : -FLT_MAX;
        tile_max = fmaxf(tile_max, p[i]);
      }
      tile_max = rows_max(tile_max);
      const float m_new = fmaxf(m, tile_max);
      corr = __builtin_amdgcn_exp2f(m - m_new);
      m = m_new;
      // a masked score is -FLT_MAX: its weight is 0 unless the row has seen nothing yet
      // (m_new is then -FLT_MAX too), which the test catches
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        p[i] = (p[i] > -FLT_MAX) ? __builtin_amdgcn_exp2f(p[i] - m_new) : 0.f;
        sum += p[i];
      }
    }
    l = l * corr + sum;   // this lane's share of the row's sum; the four lanes of a row meet at the end
    bf16x8 pf[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const uint4 w = make_uint4(pack_bf16x2(p[8 * half], p[8 * half + 1]), pack_bf16x2(p[8 * half + 2], p[8 * half + 3]),
                                 pack_bf16x2(p[8 * half + 4], p[8 * half + 5]), pack_bf16x2(p[8 * half + 6], p[8 * half + 7]));
      pf[half] = __builtin_bit_cast(bf16x8, w);
    }
    // O^T += V^T P^T, one MFMA per 32-key half
#pragma unroll
    for (int nt = 0; nt < DT; ++nt) {
      o[nt] *= corr;
      const bf16_t* vrow = &Vt[(nt * 16 + c16) * VROW];
      const int sw = ((nt * 2 + (c16 >> 3)) & 7) << 2;   // this row's permutation of its four-key groups
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const uint2 lo = *reinterpret_cast<const uint2*>(vrow + ((half * 32 + g * 4) ^ sw));
        const uint2 hi = *reinterpret_cast<const uint2*>(vrow + ((half * 32 + 16 + g * 4) ^ sw));
        const uint4 vv = make_uint4(lo.x, lo.y, hi.x, hi.y);
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vv), pf[half], o[nt], 0, 0, 0);
      }
    }
    }
  }

  l = RW == 32 ? halves_sum(l) : rows_sum(l);
  if (TEAMS > 1) {
    // the other teams leave their states where their tiles were; team 0 adds them in team order
    __syncthreads();      // every tile has been read
    float* state = reinterpret_cast<float*>(team_room + team * kTeamBytes) + tid * (OV * OT + 2);
    if (team > 0) {
      state[0] = m;
      state[1] = l;
#pragma unroll
      for (int nt = 0; nt < OT; ++nt)
#pragma unroll
        for (int e = 0; e < OV; e += 2) *reinterpret_cast<float2*>(state + 2 + OV * nt + e) = make_float2(o[nt][e], o[nt][e + 1]);
    }
    __syncthreads();
    if (team == 0) {
      float big = m;
#pragma unroll
      for (int k = 1; k < TEAMS; ++k) big = fmaxf(big, state[k * (kTeamBytes / 4)]);
      const float e0 = __builtin_amdgcn_exp2f(m - big);
      l *= e0;
#pragma unroll
      for (int nt = 0; nt < OT; ++nt) o[nt] *= e0;
#pragma unroll
      for (int k = 1; k < TEAMS; ++k) {
        const float* other = state + k * (kTeamBytes / 4);
        const float e = __builtin_amdgcn_exp2f(other[0] - big);
        l += other[1] * e;
#pragma unroll
        for (int nt = 0; nt < OT; ++nt)
#pragma unroll
          for (int x = 0; x < OV; x += 2) {
            const float2 theirs = *reinterpret_cast<const float2*>(other + 2 + OV * nt + x);
            o[nt][x] += theirs.x * e;
            o[nt][x + 1] += theirs.y * e;
          }
      }
    }
  }
  if (row_ok && team == 0) {
    const float inv = 1.f / l;
    bf16_t* dst = out + static_cast<int64_t>(row0 + my_row) * out_stride + static_cast<int64_t>(head) * d;
#pragma unroll
    for (int nt = 0; nt < OT; ++nt) {
#pragma unroll
      for (int j = 0; j < OV / 4; ++j) {    // four consecutive channels
        uint2 w;
        w.x = pack_bf16x2(o[nt][4 * j] * inv, o[nt][4 * j + 1] * inv);
        w.y = pack_bf16x2(o[nt][4 * j + 2] * inv, o[nt][4 * j + 3] * inv);
        const int c = RW == 32 ? nt * 32 + 8 * j + 4 * h : nt * 16 + g * 4;
        if (RW == 16 || c < d) *reinterpret_cast<uint2*>(dst + c) = w;
      }
    }
  }
  }  // runs of this block
}

}  // namespace alofa

using namespace alofa;

// Teams per block: as many as the registers (128 per lane with 1,024 threads, and no spills) and the LDS of a
// compute unit hold at this head size.
template <int DT>
constexpr int kTeams = (DT <= 2 || DT == 4) ? 4 : DT <= 8 ? 2 : 1;
// ... where the heads of a group share the tiles: teams of as many waves as the block serves heads (six to eight)
// (two teams of seven waves of head size 64 would spill)
template <int DT>
constexpr int kShareTeams = DT <= 2 ? 2 : 1;

// How many heads of a group share their tiles in one block (0: none do; every head has blocks of its own). A
// shared tile serves 16 rows of each of these heads where an unshared one serves 64 rows of one head, so fewer
// than six heads save no staging (measured: five lose a fifth at 40/8 heads of size 128 and 16k keys, seven
// win an eighth to a fifth at 28/4). Larger groups go in equal chunks of at most eight heads. Sharing cuts a
// run of 64 rows into four blocks of 16, each of which walks the run's tiles with fewer teams: it pays when
// there are enough blocks to fill the chip twice anyway, and loses when the longest block's walk is what the
// launch waits for. Eight waves of head size 256 would not keep their state in registers.
extern "C" int alofa_attention_prefill_share(int heads, int kv_heads, int d, int runs, int compute_units) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || d > 128) return 0;
  const int group = heads / kv_heads, chunks = (group + 7) / 8, width = (group + chunks - 1) / chunks;
  if (width < 6) return 0;
  const int64_t blocks = static_cast<int64_t>(runs) * kv_heads * chunks * 4;
  return blocks >= 2 * static_cast<int64_t>(compute_units) ? width : 0;
}

// Query rows per wave: 32 where `share` heads of a group share their tiles and the head size is a multiple of
// 32 up to 96 (measured, 14/2 heads of size 64, prompts of 2,048 tokens: three 72 against 103 us, four 76 against
// 105, eight 144 against 207; 12/2 of size 96, four prompts: 91 against 121; 16/2 of size 32: 57 against 70), else
// 16: at head size 128 the state of 32 rows does not fit a wave's registers beside the tile on its way (40/8
// heads, 16k keys: 4.3 against 1.6 ms), and where every head has blocks of its own the two forms time alike
// (14/2 heads of size 64, 2,048 tokens: 32.9 against 32.1 us). Blocks of 32 rows are half as many and a compute
// unit holds one of them: below one and a half blocks per compute unit the 16-row form's smaller blocks spread
// prompts' unequal runs better (two prompts of 2,048 tokens: 64 against 56 us; one of 4,096: 117 against 100).
// At head size 128 the state of 32 rows fits beside a tile of 32 keys on its way (tiles of 64: spills, 4.3 against
// 1.6 ms for 40/8 heads and 16k keys): where every head has blocks of its own, a block of two teams of two waves,
// in launches of at least two blocks per compute unit (40/8 heads, 2,048 rows: 133 against 146 us at 2,048 keys,
// 1.56 against 1.67 ms at 16k; 4,096 rows at 16k: 2.33 against 2.60 ms; with fewer blocks the four-wave blocks
// leave compute units idle, 16/16 heads and 2,048 rows: 65 against 56 us); with shared tiles it gains 1 to 3 %
// and is left out.
extern "C" int alofa_attention_prefill_rows_fit(int d, int share) {
  return share > 0 ? (d % 32 == 0 && d <= 96) : d == 128;
}
extern "C" int alofa_attention_prefill_rows(int heads, int kv_heads, int d, int share, int runs, int compute_units) {
  if (!alofa_attention_prefill_rows_fit(d, share) || heads <= 0 || kv_heads <= 0) return 16;
  if (share == 0) return static_cast<int64_t>(runs) * heads >= 4 * static_cast<int64_t>(compute_units) ? 32 : 16;   // (two runs a block)
  const int group = heads / kv_heads, chunks = (group + share - 1) / share;
  return static_cast<int64_t>(runs) * kv_heads * chunks * 2 * 2 >= 3 * static_cast<int64_t>(compute_units) ? 32 : 16;
}

extern "C" int alofa_attention_prefill_supports(int d) {
  return d == 16 || d == 32 || d == 48 || d == 64 || d == 96 || d == 128 || d == 256;
}

extern "C" int alofa_attention_prefill(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                       const void* k_cache, const void* v_cache, const int32_t* block_table,
                                       int max_blocks, const int32_t* tiles, int n_tiles, int heads, int kv_heads, int d,
                                       int block_size, int window, float scale, int share, int rows_per_wave, hipStream_t stream) {
  ALOFA_REQUIRE(n_tiles > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
                "attention_prefill: tiles=%d heads=%d kv_heads=%d (kv_heads must divide heads)", n_tiles, heads, kv_heads);
  ALOFA_REQUIRE(alofa_attention_prefill_supports(d), "attention_prefill: head size %d is not built (16, 32, 48, 64, 96, 128, 256 are)", d);
  ALOFA_REQUIRE(block_size >= 8 && (block_size & (block_size - 1)) == 0 && max_blocks > 0 && window >= 0,
                "attention_prefill: block_size=%d must be a power of two, at least 8; max_blocks=%d window=%d", block_size, max_blocks, window);
  int bs_shift = 0;
  while ((1 << bs_shift) < block_size) ++bs_shift;
  ALOFA_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0,
                "attention_prefill: q rows must be 16-byte aligned and out rows 8-byte aligned");
  const int group = heads / kv_heads, width = share;
  ALOFA_REQUIRE(width == 0 || (width >= 6 && width <= 8 && d <= 128 && width <= group),
                "attention_prefill: %d heads of a group of %d cannot share their tiles at head size %d (six to eight can, up to size 128)",
                width, group, d);
  const int chunks = width ? (group + width - 1) / width : 0;
  ALOFA_REQUIRE(rows_per_wave == 16 || (rows_per_wave == 32 && alofa_attention_prefill_rows_fit(d, width)),
                "attention_prefill: %d rows a wave at head size %d with %d heads sharing their tiles (16 always; 32 with shared tiles and head sizes 32, 64, 96, and without at head size 128)",
                rows_per_wave, d, width);
#define ALOFA_PREFILL_AS(DT, TEAMS, WPT, SHARE, GRID)                                                                         \
  attention_prefill_kernel<DT, TEAMS, WPT, SHARE><<<GRID, 64 * WPT * TEAMS, 0, stream>>>(                                    \
      static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(k_cache), \
      static_cast<const bf16_t*>(v_cache), block_table, max_blocks, tiles, heads, kv_heads, bs_shift, window, scale)
#define ALOFA_PREFILL_AS32(DT, TEAMS, WPT, SHARE, GRID)                                                                       \
  attention_prefill_kernel<DT, TEAMS, WPT, SHARE, 32, (DT > 6 ? 32 : 64)><<<GRID, 64 * WPT * TEAMS, 0, stream>>>(            \
      static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(k_cache), \
      static_cast<const bf16_t*>(v_cache), block_table, max_blocks, tiles, heads, kv_heads, bs_shift, window, scale)
#define ALOFA_PREFILL_WIDE32(DT, WPT)                                                                            \
  if (width == WPT) ALOFA_PREFILL_AS32(DT, (kShareTeams<DT>), WPT, true, dim3(n_tiles, kv_heads * chunks, 2))
#define ALOFA_PREFILL32(DT)                                                                         \
  ALOFA_PREFILL_WIDE32(DT, 8); else ALOFA_PREFILL_WIDE32(DT, 7); else ALOFA_PREFILL_WIDE32(DT, 6)
#define ALOFA_PREFILL_WIDE(DT, WPT)                                                                            \
  if (width == WPT && DT <= 8) ALOFA_PREFILL_AS((DT <= 8 ? DT : 8), (kShareTeams<(DT <= 8 ? DT : 8)>), WPT, true, dim3(n_tiles, kv_heads * chunks, 4))
#define ALOFA_PREFILL(DT)                                                                         \
  ALOFA_PREFILL_WIDE(DT, 8); else ALOFA_PREFILL_WIDE(DT, 7); else ALOFA_PREFILL_WIDE(DT, 6);   \
  else ALOFA_PREFILL_AS(DT, kTeams<DT>, 4, false, dim3(n_tiles, heads))
  if (rows_per_wave == 32) {
    switch (d / 16) {
      case 2: ALOFA_PREFILL32(2); break;
      case 4: ALOFA_PREFILL32(4); break;
      case 6: ALOFA_PREFILL32(6); break;
      case 8: ALOFA_PREFILL_AS32(8, 2, 2, false, dim3(n_tiles, heads)); break;
    }
    return check_launch("attention_prefill");
  }
  switch (d / 16) {
    case 1: ALOFA_PREFILL(1); break;
    case 2: ALOFA_PREFILL(2); break;
    case 3: ALOFA_PREFILL(3); break;
    case 4: ALOFA_PREFILL(4); break;
    case 6: ALOFA_PREFILL(6); break;
    case 8: ALOFA_PREFILL(8); break;
    case 16: ALOFA_PREFILL(16); break;
  }
#undef ALOFA_PREFILL
#undef ALOFA_PREFILL_WIDE
#undef ALOFA_PREFILL32
#undef ALOFA_PREFILL_WIDE32
#undef ALOFA_PREFILL_AS32
#undef ALOFA_PREFILL_AS
  return check_launch("attention_prefill");
}
