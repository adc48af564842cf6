// Paged grouped-query attention for few query tokens per request (decode steps
// and short portions), bfloat16 on MFMA. The work is reading every visible key
// and value once, so all query heads of one key head (up to 16) are served
// together: they are the 16 columns of the matrix-core tiles.
//
// A block of NW wavefronts handles (token, key head, part): every wave a
// contiguous share of the token's visible keys, in tiles of 16 keys that start
// at multiples of 16, two tiles per step. Both products are taken transposed,
// so that a lane's data stays with one query head (v_mfma_f32_16x16x32_bf16;
// lane l: A row and B column l % 16, the 8 reduction slots 8 * (l / 16) .. + 7,
// D column l % 16 and rows 4 * (l / 16) .. + 3):
//   S^T[key, head] = K[key, :] . Q[head, :]        A = keys straight from the cache, B = queries (registers)
//   O^T[c, head]  += V^T[c, key] * P^T[key, head]   A = values straight from the cache, B = weights (registers)
// The cache holds the values transposed, so four consecutive keys of a channel
// are one 8-byte load. After the first product of a step lane l holds, for head
// l % 16, the scores of keys 4 g + r of either tile (g = l / 16, r = 0..3); these
// eight are its reduction slots of the second product when the values are read
// in the same order, so the weights never leave their registers. Scores, the
// running maximum, the weights and their sum are float (in units of log2 e);
// the weights are rounded to bfloat16 only as MFMA operands.
//
// The pages of a wave's share are read from the block table once, 64 at a time,
// one per lane; keys and values of the next two steps are on their way while a
// step is computed. At the end the waves' states meet in LDS and are combined in
// wave order. A block reads its keys at the rate of one compute unit, so where
// the (token, key head) pairs are far fewer than the compute units their keys
// are cut into parts, one block each. Few parts hand their states over in the
// library's workspace (uncached memory and a counter): the block that arrives
// last combines them in part order. Many parts leave them in a scratch buffer
// and a second kernel combines them (the last block's work grows with the parts,
// the second kernel's does not).
// The order of additions depends only on the key range, the wave count and the
// part count, never on timing.
// Cache layout: keys [block, kv_head, slot_in_block, d], values transposed [block, kv_head, d, slot_in_block].
#include "common.h"

#include <type_traits>

#include <float.h>

namespace alofa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kMaxSplits = 64;
constexpr int kHeadsPerBlock = 16;   // query heads of one key head that a block serves (the columns of a tile)

// What the kernel needs to take the new token's projections as they come out of the fused query / key / value
// product (kRope): q then points to rows [queries | keys | values] that are not yet rotated, one token per
// request; the queries and the new key are rotated here by the token's position (half-split pairing,
// cos / sin: [position, d / 2]), the new key and value are used from registers and written to the token's
// cache slot by the one wave that owns the last tile of keys. Needs d a multiple of 64 (a channel and its
// partner lie in the same lane's fragments).
struct RopeArgs {
  const float* cos_t;
  const float* sin_t;
  const int64_t* slots;
};

struct Pair8 {
  uint4 lo, hi;
};

// a (low half) and b (high half) of eight pairs, rotated
__device__ __forceinline__ Pair8 rotate8(uint4 lo, uint4 hi, float4 c_lo, float4 c_hi, float4 s_lo, float4 s_hi) {
#pragma clang fp contract(off)
  const uint32_t a[4] = {lo.x, lo.y, lo.z, lo.w}, b[4] = {hi.x, hi.y, hi.z, hi.w};
  const float cs[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
  const float sn[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
  uint32_t ra[4], rb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a0 = __uint_as_float(a[i] << 16), a1 = __uint_as_float(a[i] & 0xffff0000u);
    const float b0 = __uint_as_float(b[i] << 16), b1 = __uint_as_float(b[i] & 0xffff0000u);
    ra[i] = pack_bf16x2(a0 * cs[2 * i] - b0 * sn[2 * i], a1 * cs[2 * i + 1] - b1 * sn[2 * i + 1]);
    rb[i] = pack_bf16x2(b0 * cs[2 * i] + a0 * sn[2 * i], b1 * cs[2 * i + 1] + a1 * sn[2 * i + 1]);
  }
  return Pair8{make_uint4(ra[0], ra[1], ra[2], ra[3]), make_uint4(rb[0], rb[1], rb[2], rb[3])};
}

// DT = d / 16; NW: waves per block. blockIdx.y = key head * chunks + chunk of up to 16 heads of its group.
template <int DT, int NW, bool kRope>
__global__ void __launch_bounds__(64 * NW) attention_decode_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, float* __restrict__ partial, const bf16_t* __restrict__ q,
    int64_t q_stride, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ req_of_token,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ rows, int heads, int kv_heads,
    int bs_shift, int window, float scale, RopeArgs rope, int* __restrict__ counters) {
  static_assert(!kRope || DT % 4 == 0, "the rotation needs a channel and its partner in the same lane: d a multiple of 64");
  constexpr int d = DT * 16;
  constexpr int DS = (d + 31) / 32;            // steps of 32 along d in the first product
  // per wave and head: maximum, sum of weights, (two unused,) weighted value sums of the wave's share
  __shared__ __attribute__((aligned(16))) float state[NW][kHeadsPerBlock][d + 4];
  __shared__ int last_block;
  const int group = heads / kv_heads;
  const int chunks = (group + kHeadsPerBlock - 1) / kHeadsPerBlock;
  // the tokens served are rows[0..gridDim.x) of the packed batch, or all of it
  const int t = rows ? rows[blockIdx.x] : blockIdx.x;
  const int hk = blockIdx.y / chunks, h0 = (blockIdx.y % chunks) * kHeadsPerBlock;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int c16 = lane % 16, g = lane / 16;
  const int n_parts = gridDim.z, n_splits = n_parts * NW, split = blockIdx.z * NW + wave;
  // The chain of dependent loads is what a short context's attention takes its time from: position and request ->
  // pages -> keys. With one token per request the request is the token's own number (req_of_token may be null
  // then), and the first 64 pages of its table set out at once, before the position says which pages are needed.
  const int32_t* table = block_table + static_cast<int64_t>(req_of_token ? req_of_token[t] : t) * max_blocks;
  int my_page = table[lane < max_blocks ? lane : max_blocks - 1];
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  // the visible keys lo..p lie in the 16-key tiles first..last; a wave takes a contiguous run of tiles
  const int first = lo >> 4, last = p >> 4;
  const int per_split = (last - first + 1 + n_splits - 1) / n_splits;
  const int tile_begin = first + split * per_split;
  const int tile_end = (tile_begin + per_split < last + 1) ? tile_begin + per_split : last + 1;
  const int bs_mask = (1 << bs_shift) - 1;

  // this lane's head and its fragments of Q (heads beyond the group: zeros)
  const bool head_ok = h0 + c16 < group;
  const int head = hk * group + (head_ok ? h0 + c16 : 0);
  bf16x8 qf[DS];
#pragma unroll
  for (int ds = 0; ds < DS; ++ds) {
    uint4 v = make_uint4(0, 0, 0, 0);
    const int c = ds * 32 + g * 8;
    if (head_ok && c < d) v = *reinterpret_cast<const uint4*>(q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(head) * d + c);
    qf[ds] = __builtin_bit_cast(bf16x8, v);
  }

  // the new token's key (this lane's channel slices, rotated) and value (channels 16 nt + c16), kRope only
  uint4 new_k[DS];
  uint32_t new_v[DT];
  float4 cs[kRope ? DS / 2 : 1][2], sn[kRope ? DS / 2 : 1][2];
  int64_t new_slot = 0;
  if constexpr (kRope) {
    new_slot = rope.slots[t];
    const bf16_t* row = q + static_cast<int64_t>(t) * q_stride;
    const bf16_t* k_row = row + static_cast<int64_t>(heads + hk) * d;
    const bf16_t* v_row = row + static_cast<int64_t>(heads + kv_heads + hk) * d;
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) new_k[ds] = *reinterpret_cast<const uint4*>(k_row + ds * 32 + g * 8);
#pragma unroll
    for (int nt = 0; nt < DT; ++nt) new_v[nt] = v_row[nt * 16 + c16];
    // (cos and sin of the pairs (c, c + d / 2): slices ds and ds + DS / 2 of this lane)
#pragma unroll
    for (int ds = 0; ds < DS / 2; ++ds) {
      const int64_t at = static_cast<int64_t>(p) * (d / 2) + ds * 32 + g * 8;
      cs[ds][0] = *reinterpret_cast<const float4*>(rope.cos_t + at), cs[ds][1] = *reinterpret_cast<const float4*>(rope.cos_t + at + 4);
      sn[ds][0] = *reinterpret_cast<const float4*>(rope.sin_t + at), sn[ds][1] = *reinterpret_cast<const float4*>(rope.sin_t + at + 4);
    }
  }

  f32x4 o[DT];
#pragma unroll
  for (int nt = 0; nt < DT; ++nt) o[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -FLT_MAX, l = 0.f;
  const float scale2 = scale * 1.44269504088896340736f;   // scores in units of log2(e)

  // lane x holds the page of logical block page_base + x; a step's keys lie within 64 pages of its first
  // (a share whose first step lies within the first 64 pages uses the pages that set out at the start)
  int page_base = ((((tile_begin + 2) << 4) - 1) >> bs_shift) < 64 ? 0 : (tile_begin << 4) >> bs_shift;
  const int last_page = p >> bs_shift;
  // (pages that a window has passed read -1: they are never used, and 0 keeps every address inside the cache)
  if (page_base != 0) {     // uniform over the wave: a share that starts past the pages already on their way
    my_page = (tile_begin < tile_end && page_base + lane <= last_page) ? table[page_base + lane] : 0;
  }
  my_page = (my_page < 0 || page_base + lane > last_page) ? 0 : my_page;

  // Operands of the step that starts at tile `tile` (two tiles): keys [tile][ds], values [tile][nt]. Every
  // lane issues every load, from the nearest visible key where its own is not visible (such scores are
  // masked, such values cleared before use): with loads that are always issued the compiler can count
  // them and wait for the oldest step only, so that two later steps stay on their way.
  struct Step {
    uint4 k[2][DS];
    uint2 v[2][DT];
  };
  const int lo4 = lo & ~3, p4 = p & ~3;
  auto fetch = [&](int tile, Step& s) __attribute__((always_inline)) {
    if ((((((tile + 2) << 4) - 1)) >> bs_shift) - page_base >= 64 && (tile << 4) <= p) {     // uniform over the wave
      page_base = (tile << 4) >> bs_shift;
      my_page = (page_base + lane <= last_page) ? table[page_base + lane] : 0;
      my_page = my_page < 0 ? 0 : my_page;
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      // the key of this lane's row of K, and the first of this lane's four keys of V^T, brought into lo..p
      int key = ((tile + kt) << 4) + c16, key4 = ((tile + kt) << 4) + 4 * g;
      key = key < lo ? lo : (key > p ? p : key);
      key4 = key4 < lo4 ? lo4 : (key4 > p4 ? p4 : key4);
      // (a step past the end of the share may lie before the window of pages held in the lanes: its operands are not used)
      const int kpage = (key >> bs_shift) - page_base, vpage = (key4 >> bs_shift) - page_base;
      const int64_t kblk = __shfl(my_page, kpage < 0 ? 0 : (kpage > 63 ? 63 : kpage), 64);
      const int64_t vblk = __shfl(my_page, vpage < 0 ? 0 : (vpage > 63 ? 63 : vpage), 64);
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        const int c = ds * 32 + g * 8;
        s.k[kt][ds] = *reinterpret_cast<const uint4*>(k_cache + ((((kblk * kv_heads + hk) << bs_shift) + (key & bs_mask)) * d) + (c < d ? c : 0));
      }
#pragma unroll
      for (int nt = 0; nt < DT; ++nt)
        s.v[kt][nt] = *reinterpret_cast<const uint2*>(v_cache + ((((vblk * kv_heads + hk) * d + nt * 16 + c16) << bs_shift) + (key4 & bs_mask)));
    }
  };

  // one step: the running state takes the two tiles from `tile` on (tiles past the share's end change nothing)
  auto compute = [&](int tile, Step& st) __attribute__((always_inline)) {
    // S^T of the two tiles (channels beyond d, in the last step of 32 of a head size that is no multiple of 32,
    // meet zeros of Q)
    // Most steps of a long context touch neither end of the visible keys nor the new token: they skip the masks and
    // the new token's insertion (branches of the whole wave with no loads inside; the results are the same bits).
    const bool last_here = kRope && tile + 1 >= last;                                                   // the step holds the new token's tile
    const bool inner = (tile << 4) >= lo && (((tile + 2) << 4) - 1) <= p && tile + 1 < tile_end;        // every key of the step is seen
    f32x4 s[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
      // (kRope: the new token's key is not in the cache yet: its row of the last tile comes from the registers)
      const bool new_row = last_here && tile + kt == last && c16 == (p & 15);
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        uint4 kf = st.k[kt][ds];
        if (last_here) {      // (word by word: a choice between two whole operands would be made through memory)
          kf.x = new_row ? new_k[ds].x : kf.x;
          kf.y = new_row ? new_k[ds].y : kf.y;
          kf.z = new_row ? new_k[ds].z : kf.z;
          kf.w = new_row ? new_k[ds].w : kf.w;
        }
        s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf), qf[ds], s[kt], 0, 0, 0);
      }
    }
    // scale, mask, running maximum; the four lanes of a head agree on the maximum
    float pw[8];
    float step_max = -FLT_MAX;
    if (inner) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        pw[i] = s[i / 4][i % 4] * scale2;
        step_max = fmaxf(step_max, pw[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int key = ((tile + i / 4) << 4) + 4 * g + i % 4;
        const bool seen = key >= lo && key <= p && tile + i / 4 < tile_end;
        pw[i] = seen ? s[i / 4][i % 4] * scale2 : -FLT_MAX;
        step_max = fmaxf(step_max, pw[i]);
      }
    }
    step_max = rows_max(step_max);
    const float m_new = fmaxf(m, step_max);
    const float corr = __builtin_amdgcn_exp2f(m - m_new);    // 1 while nothing was seen yet (both -FLT_MAX)
    m = m_new;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pw[i] = (inner || pw[i] > -FLT_MAX) ? __builtin_amdgcn_exp2f(pw[i] - m_new) : 0.f;
      sum += pw[i];
    }
    l = l * corr + sum;   // this lane's share of the head's sum; the four lanes of a head meet at the end
    const uint4 w = make_uint4(pack_bf16x2(pw[0], pw[1]), pack_bf16x2(pw[2], pw[3]), pack_bf16x2(pw[4], pw[5]), pack_bf16x2(pw[6], pw[7]));
    const bf16x8 pf = __builtin_bit_cast(bf16x8, w);
    // What lies beyond the visible keys is not data: it is cleared, so that a weight of zero times it is zero.
    // (Within lo..p a weight of zero meets a visible key's values.)
    uint32_t keep_x[2] = {0xffffffffu, 0xffffffffu}, keep_y[2] = {0xffffffffu, 0xffffffffu};
    if (!inner) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const int key4 = ((tile + kt) << 4) + 4 * g;
        const int lo_e = lo - key4, hi_e = p - key4 + 1;       // elements lo_e .. hi_e - 1 are visible
        keep_x[kt] = ((0 < lo_e || 0 >= hi_e) ? 0u : 0x0000ffffu) | ((1 < lo_e || 1 >= hi_e) ? 0u : 0xffff0000u);
        keep_y[kt] = ((2 < lo_e || 2 >= hi_e) ? 0u : 0x0000ffffu) | ((3 < lo_e || 3 >= hi_e) ? 0u : 0xffff0000u);
      }
    }
    // O^T += V^T P^T
#pragma unroll
    for (int nt = 0; nt < DT; ++nt) {
      o[nt] *= corr;
      uint32_t vw[4] = {st.v[0][nt].x & keep_x[0], st.v[0][nt].y & keep_y[0], st.v[1][nt].x & keep_x[1], st.v[1][nt].y & keep_y[1]};
      if (last_here) {
        // the new token's value takes its place among this lane's four keys of the last tile
#pragma unroll
        for (int w2 = 0; w2 < 4; ++w2) {
          const bool hit = tile + w2 / 2 == last && g == ((p & 15) >> 2) && ((p & 3) >> 1) == (w2 & 1);
          const uint32_t ins = (p & 1) ? ((vw[w2] & 0x0000ffffu) | (new_v[nt] << 16)) : ((vw[w2] & 0xffff0000u) | new_v[nt]);
          vw[w2] = hit ? ins : vw[w2];
        }
      }
      const uint4 vv = make_uint4(vw[0], vw[1], vw[2], vw[3]);
      o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vv), pf, o[nt], 0, 0, 0);
    }
  };

  // Three steps (two for large heads, whose operands fill the registers) are on their way or in work: each
  // set of registers is filled again as soon as its step is done (no copies between sets: a copy would
  // wait for the load).
  constexpr bool kThree = DT <= 5;
  constexpr int kStride = kThree ? 6 : 4;
  Step s0, s1, s2;
  int tile = tile_begin;
  if (tile < tile_end) fetch(tile, s0);
  if (tile + 2 < tile_end) fetch(tile + 2, s1);
  if (kThree && tile + 4 < tile_end) fetch(tile + 4, s2);
  // The rotation comes after the first keys and values have set out: it needs cos and sin only, which were
  // asked for before them.
  if constexpr (kRope) {
    // pairs (c, c + d / 2): slices ds and ds + DS / 2 of this lane
#pragma unroll
    for (int ds = 0; ds < DS / 2; ++ds) {
      const float4 c_lo = cs[ds][0], c_hi = cs[ds][1], s_lo = sn[ds][0], s_hi = sn[ds][1];
      const Pair8 rq = rotate8(__builtin_bit_cast(uint4, qf[ds]), __builtin_bit_cast(uint4, qf[ds + DS / 2]), c_lo, c_hi, s_lo, s_hi);
      qf[ds] = __builtin_bit_cast(bf16x8, rq.lo);
      qf[ds + DS / 2] = __builtin_bit_cast(bf16x8, rq.hi);
      const Pair8 rk = rotate8(new_k[ds], new_k[ds + DS / 2], c_lo, c_hi, s_lo, s_hi);
      new_k[ds] = rk.lo;
      new_k[ds + DS / 2] = rk.hi;
    }
    // the wave that owns the last tile of keys (in the first chunk of heads) writes the token's cache slot
    if (h0 == 0 && tile_begin <= last && last < tile_end) {
      const int64_t blk = new_slot >> bs_shift, off = new_slot & bs_mask;
      if (c16 == 0) {
#pragma unroll
        for (int ds = 0; ds < DS; ++ds)
          *reinterpret_cast<uint4*>(k_cache + ((((blk * kv_heads + hk) << bs_shift) + off) * d) + ds * 32 + g * 8) = new_k[ds];
      }
      if (g == 0) {
#pragma unroll
        for (int nt = 0; nt < DT; ++nt)
          v_cache[(((blk * kv_heads + hk) * d + nt * 16 + c16) << bs_shift) + off] = static_cast<bf16_t>(new_v[nt]);
      }
    }
  }

  // while every set has a further step to fetch: no branches, so that the waits are counted exactly
  for (; tile + 2 * kStride - 2 < tile_end; tile += kStride) {
    compute(tile, s0);
    fetch(tile + kStride, s0);
    compute(tile + 2, s1);
    fetch(tile + 2 + kStride, s1);
    if (kThree) {
      compute(tile + 4, s2);
      fetch(tile + 4 + kStride, s2);
    }
  }
  // the last steps: nothing is fetched that no step will use (a wave ends only when its loads have come back)
  for (; tile < tile_end; tile += kStride) {
    compute(tile, s0);
    if (tile + kStride < tile_end) fetch(tile + kStride, s0);
    if (tile + 2 < tile_end) compute(tile + 2, s1);
    if (tile + 2 + kStride < tile_end) fetch(tile + 2 + kStride, s1);
    if (kThree) {
      if (tile + 4 < tile_end) compute(tile + 4, s2);
      if (tile + 4 + kStride < tile_end) fetch(tile + 4 + kStride, s2);
    }
  }
  l = rows_sum(l);

  // the wave's state: head c16; this lane holds channels 16 nt + 4 g + r
  {
    float* mine = state[wave][c16];
    if (g == 0) { mine[0] = m; mine[1] = l; }
#pragma unroll
    for (int nt = 0; nt < DT; ++nt) *reinterpret_cast<f32x4*>(mine + 4 + nt * 16 + 4 * g) = o[nt];
  }
  __syncthreads();

  // the waves' states are combined in wave order; thread x takes channel x % d of head x / d
  for (int x = threadIdx.x; x < kHeadsPerBlock * d; x += 64 * NW) {
    const int i = x / d, c = x % d;
    if (h0 + i >= group) break;
    const int h = hk * group + h0 + i;
    float big = state[0][i][0];
#pragma unroll
    for (int w = 1; w < NW; ++w) big = fmaxf(big, state[w][i][0]);
    float total = 0.f, acc = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float e = __builtin_amdgcn_exp2f(state[w][i][0] - big);
      total += state[w][i][1] * e;
      acc += state[w][i][4 + c] * e;
    }
    if (n_parts == 1) {
      store_f32(out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * d + c, acc / total);
    } else {
      float* dst = partial + ((static_cast<int64_t>(blockIdx.x) * heads + h) * n_parts + blockIdx.z) * (d + 2);
      if (counters) {   // (device scope: written through to memory, where blocks on every die find it)
        __hip_atomic_store(dst + 2 + c, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (c == 0) {
          __hip_atomic_store(dst, big, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(dst + 1, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else {
        dst[2 + c] = acc;
        if (c == 0) { dst[0] = big; dst[1] = total; }
      }
    }
  }
  if (n_parts == 1 || !counters) return;

  // The parts of a (token, key head) hand their states over in the library's workspace: every wave waits
  // until its stores have been performed in memory, then the block is counted; the block that arrives last
  // combines all parts in part order (the same sum on every run) and puts the counter back to zero.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) {
    int* counter = counters + blockIdx.x * gridDim.y + blockIdx.y;
    const int arrived = atomicAdd(counter, 1);
    last_block = arrived == n_parts - 1;
    if (last_block) atomicExch(counter, 0);
  }
  __syncthreads();
  if (!last_block) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  for (int x = threadIdx.x; x < kHeadsPerBlock * d; x += 64 * NW) {
    const int i = x / d, c = x % d;
    if (h0 + i >= group) break;
    const int h = hk * group + h0 + i;
    const float* src = partial + (static_cast<int64_t>(blockIdx.x) * heads + h) * n_parts * (d + 2);
    float big = -FLT_MAX, total = 0.f, acc = 0.f;
    if (n_parts <= 16) {
      // up to sixteen parts: everything that is read is asked for at once (the states come from memory; one after
      // the other, every load is waited for by itself), in arrays of four, eight or sixteen; same sums in the same
      // order as below
      auto at_once = [&](auto count) {
        constexpr int kCount = decltype(count)::value;
        float ms[kCount], ls[kCount], vs[kCount];
#pragma unroll
        for (int u = 0; u < kCount; ++u) {
          const float* part = src + min(u, n_parts - 1) * (d + 2);
          ms[u] = __hip_atomic_load(part, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ls[u] = __hip_atomic_load(part + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          vs[u] = __hip_atomic_load(part + 2 + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < kCount; ++u)
          if (u < n_parts) big = fmaxf(big, ms[u]);
#pragma unroll
        for (int u = 0; u < kCount; ++u)
          if (u < n_parts) {
            const float e = __builtin_amdgcn_exp2f(ms[u] - big);
            total += ls[u] * e;
            acc += vs[u] * e;
          }
      };
      if (n_parts <= 4) at_once(std::integral_constant<int, 4>());
      else if (n_parts <= 8) at_once(std::integral_constant<int, 8>());
      else at_once(std::integral_constant<int, 16>());
    } else {
      for (int sp = 0; sp < n_parts; ++sp) big = fmaxf(big, __hip_atomic_load(src + sp * (d + 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
#pragma unroll 4
      for (int sp = 0; sp < n_parts; ++sp) {
        const float* part = src + sp * (d + 2);
        const float e = __builtin_amdgcn_exp2f(__hip_atomic_load(part, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - big);
        total += __hip_atomic_load(part + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * e;
        acc += __hip_atomic_load(part + 2 + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * e;
      }
    }
    store_f32(out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * d + c, acc / total);
  }
}

// Combines the parts' states of one (token, head) (maxima in units of log2 e). The waves of the block take the
// parts in turn (wave w parts w, w + waves, ..), sixteen at a time with all their loads on their way together:
// the states come from memory, and one after the other 64 parts took 20 us. Every wave sums its parts in
// ascending order and the waves' sums are added in wave order, so the result depends on nothing but the number
// of parts and of waves.
__global__ void __launch_bounds__(256) attention_merge_kernel(bf16_t* __restrict__ out, int64_t out_stride,
                                                              const float* __restrict__ partial,
                                                              const int32_t* __restrict__ rows, int heads, int d,
                                                              int n_splits) {
  __shared__ float sums[4][256];
  const int t = rows ? rows[blockIdx.x] : blockIdx.x, h = blockIdx.y, lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64, waves = blockDim.x / 64;
  const float* src = partial + (static_cast<int64_t>(blockIdx.x) * heads + h) * n_splits * (d + 2);
  // lane s holds part s's maximum and sum (n_splits <= 64)
  const float m = lane < n_splits ? src[lane * (d + 2)] : -FLT_MAX;
  const float l = lane < n_splits ? src[lane * (d + 2) + 1] : 0.f;
  const float big = wave_max(m);
  const float e = __builtin_amdgcn_exp2f(m - big);
  const float total = wave_sum(l * e);
  // every lane takes part in every round, so that the weights can be read from all 64 lanes
  for (int c0 = 0; c0 < d; c0 += 64) {
    const int c = c0 + lane;
    float acc = 0.f;
    for (int base = wave; base < n_splits; base += 16 * waves) {    // uniform over the wave
      float v[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int sp = base + i * waves;
        v[i] = (sp < n_splits && c < d) ? src[sp * (d + 2) + 2 + c] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int sp = base + i * waves;
        acc += v[i] * __shfl(e, sp < n_splits ? sp : 0, 64);
      }
    }
    if (waves > 1) {
      if (c < d) sums[wave][c] = acc;
      __syncthreads();
      if (wave == 0) {
        acc = sums[0][c < d ? c : 0];
        for (int w = 1; w < waves; ++w) acc += sums[w][c < d ? c : 0];
      }
    }
    if (wave == 0 && c < d) store_f32(out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * d + c, acc / total);
  }
}

}  // namespace alofa

using namespace alofa;

// Waves per block: each takes a share of the keys; their states meet in LDS (which bounds their number). From head
// size 128 on four: a block of eight waves leaves 256 registers to a lane, which these head sizes do not fit without spills.
extern "C" int alofa_attention_decode_waves(int d) { return d < 128 ? 8 : 4; }

// Floats of scratch that n_splits > 1 needs.
extern "C" int64_t alofa_attention_decode_scratch(int tokens, int heads, int d, int n_splits) {
  return n_splits > 1 ? static_cast<int64_t>(tokens) * heads * n_splits * (d + 2) : 0;
}

// Whether the parts of these sizes fit the library's workspace (their states and a counter per (token, key head,
// chunk of heads)), so that the last block of a (token, key head) can combine them and no second kernel is needed.
extern "C" int alofa_attention_decode_can_hand_over(int tokens, int heads, int kv_heads, int d, int n_splits) {
  if (tokens <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || n_splits <= 1) return 0;
  const Workspace& ws = workspace();
  const int64_t counters = static_cast<int64_t>(tokens) * kv_heads * ((heads / kv_heads + kHeadsPerBlock - 1) / kHeadsPerBlock);
  return ws.tiles != nullptr && counters <= ws.n_counters && alofa_attention_decode_scratch(tokens, heads, d, n_splits) <= ws.tile_floats;
}

// cos_t, sin_t, slots: null for queries that are rotated and a cache that is written already; else (see RopeArgs)
// q holds rows [queries | keys | values] of one new token per request. req_of_token may be null when every
// request brings one token: token i then belongs to row i of block_table. hand_over: the parts meet in the
// workspace (alofa_attention_decode_can_hand_over must hold; `partial` is not used), not in `partial` and a second kernel.
extern "C" int alofa_attention_decode(void* out, int64_t out_stride, float* partial, const void* q, int64_t q_stride,
                                      void* k_cache, void* v_cache, const int32_t* block_table,
                                      int max_blocks, const int32_t* req_of_token, const int32_t* positions,
                                      const int32_t* rows, int tokens, int heads, int kv_heads, int d, int block_size, int window,
                                      float scale, int n_splits, const float* cos_t, const float* sin_t, const int64_t* slots,
                                      int hand_over, hipStream_t stream) {
  ALOFA_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
                "attention_decode: tokens=%d heads=%d kv_heads=%d (kv_heads must divide heads)", tokens, heads, kv_heads);
  ALOFA_REQUIRE(d >= 16 && d <= 256 && d % 16 == 0, "attention_decode: head size %d must be 16..256 in steps of 16", d);
  ALOFA_REQUIRE(block_size >= 4 && (block_size & (block_size - 1)) == 0 && max_blocks > 0 && window >= 0,
                "attention_decode: block_size=%d must be a power of two, at least 4; max_blocks=%d window=%d", block_size, max_blocks, window);
  int bs_shift = 0;
  while ((1 << bs_shift) < block_size) ++bs_shift;
  ALOFA_REQUIRE(n_splits >= 1 && n_splits <= kMaxSplits && (n_splits == 1 || partial || hand_over), "attention_decode: n_splits=%d (1..%d) needs scratch when above 1", n_splits, kMaxSplits);
  int* counters = nullptr;
  if (hand_over && n_splits > 1) {
    ALOFA_REQUIRE(alofa_attention_decode_can_hand_over(tokens, heads, kv_heads, d, n_splits),
                  "attention_decode: the states of %d parts of %d tokens do not fit the workspace", n_splits, tokens);
    partial = workspace().tiles;
    counters = workspace().counters;
  }
  ALOFA_REQUIRE(q_stride % 8 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0, "attention_decode: q rows must be 16-byte aligned");
  ALOFA_REQUIRE(reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 8 == 0, "attention_decode: caches must be 16-byte aligned");
  const bool fused = cos_t != nullptr;
  ALOFA_REQUIRE(!fused || (sin_t && slots && d % 64 == 0 && q_stride >= static_cast<int64_t>(heads + 2 * kv_heads) * d),
                "attention_decode: the rotary variant needs sin, slots, rows of queries, keys and values, and a head size in steps of 64 (d=%d)", d);
  ALOFA_REQUIRE(!fused || (reinterpret_cast<uintptr_t>(cos_t) % 16 == 0 && reinterpret_cast<uintptr_t>(sin_t) % 16 == 0), "attention_decode: cos and sin must be 16-byte aligned");
  const int group = heads / kv_heads;
  const RopeArgs rope{cos_t, sin_t, slots};
  dim3 grid(tokens, kv_heads * ((group + kHeadsPerBlock - 1) / kHeadsPerBlock), n_splits);
#define ALOFA_DECODE(DT, NW, ROPE)                                                                                        \
  attention_decode_kernel<DT, NW, ROPE><<<grid, 64 * NW, 0, stream>>>(                                                    \
      static_cast<bf16_t*>(out), out_stride, partial, static_cast<const bf16_t*>(q), q_stride,                            \
      static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), block_table, max_blocks, req_of_token,                \
      positions, rows, heads, kv_heads, bs_shift, window, scale, rope, counters)
  if (fused) {
    switch (d / 64) {
      case 1: ALOFA_DECODE(4, 8, true); break;
      case 2: ALOFA_DECODE(8, 4, true); break;
      case 3: ALOFA_DECODE(12, 4, true); break;
      default: ALOFA_DECODE(16, 4, true); break;
    }
  } else {
    switch (d / 16) {
      case 1: ALOFA_DECODE(1, 8, false); break;
      case 2: ALOFA_DECODE(2, 8, false); break;
      case 3: ALOFA_DECODE(3, 8, false); break;
      case 4: ALOFA_DECODE(4, 8, false); break;
      case 5: ALOFA_DECODE(5, 8, false); break;
      case 6: ALOFA_DECODE(6, 8, false); break;
      case 7: ALOFA_DECODE(7, 8, false); break;
      case 8: ALOFA_DECODE(8, 4, false); break;
      case 9: ALOFA_DECODE(9, 4, false); break;
      case 10: ALOFA_DECODE(10, 4, false); break;
      case 11: ALOFA_DECODE(11, 4, false); break;
      case 12: ALOFA_DECODE(12, 4, false); break;
      case 13: ALOFA_DECODE(13, 4, false); break;
      case 14: ALOFA_DECODE(14, 4, false); break;
      case 15: ALOFA_DECODE(15, 4, false); break;
      default: ALOFA_DECODE(16, 4, false); break;
    }
  }
#undef ALOFA_DECODE
  if (check_launch("attention_decode")) return 1;
  if (n_splits > 1 && !counters) {
    // (one wave up to sixteen parts, whose loads are all on their way at once; four beyond)
    attention_merge_kernel<<<dim3(tokens, heads), n_splits <= 16 ? 64 : 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, partial, rows, heads, d, n_splits);
    return check_launch("attention_merge");
  }
  return 0;
}
