// Paged grouped-query attention for few query tokens per request (decode steps
// and short portions), bfloat16. The work is reading every visible key and value
// once, so all query heads of one key head are served together.
//
// A block of NW wavefronts handles (token, key head and up to four of its query
// heads, part): every wave a contiguous share of the token's visible keys
// lo..p. d / 16 lanes share a key (16 channels each), so a wave takes
// 64 / (d / 16) keys per round with fully used 32-byte loads. The pages of a
// wave's share are read from the block table once, 64 at a time, one per lane;
// keys and values are on their way two rounds ahead. Every lane group keeps a
// running softmax of its own (maximum, sum of weights, weighted sum of its 16
// value channels, per head, all float); dot products use the packed bfloat16
// dot instruction with float accumulation. At the end the groups' states meet
// in LDS and are combined in group order, then the waves' states in wave
// order. With several parts (long contexts) the blocks' states go to a scratch
// buffer and a second kernel combines them in part order. The order of
// additions depends only on the key range, the wave count and the part count,
// never on timing.
// Cache layout: [block, kv_head, slot_in_block, d].
#include "common.h"

#include <float.h>

namespace alofa {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kMaxSplits = 64;

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

struct KeyValue {
  uint4 k0, k1, v0, v1;
};

// GC: query heads per block; blockIdx.y = key head * chunks + chunk of GC heads of its group; NW: waves per block.
template <int GC, int NW>
__global__ void __launch_bounds__(64 * NW) attention_decode_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, float* __restrict__ partial, const bf16_t* __restrict__ q,
    int64_t q_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ req_of_token,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ rows, int heads, int kv_heads, int d,
    int bs_shift, int window, float scale) {
  // per wave [kpi][d]: one head's weighted value sums of every lane group; then per wave and head
  // [d + 2]: maximum, sum of weights and weighted value sums of the wave's share
  extern __shared__ float lds[];
  const int group = heads / kv_heads;
  const int chunks = (group + GC - 1) / GC;
  // the tokens served are rows[0..gridDim.x) of the packed batch, or all of it
  const int t = rows ? rows[blockIdx.x] : blockIdx.x;
  const int hk = blockIdx.y / chunks, wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int n_parts = gridDim.z, n_splits = n_parts * NW, split = blockIdx.z * NW + wave;
  const int lpk = d / 16;          // lanes per key
  const int kpi = 64 / lpk;        // keys per round
  const int slot = lane / lpk, part = lane % lpk;
  const bool active = slot < kpi;
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int n_keys = p - lo + 1;
  const int per_split = (n_keys + n_splits - 1) / n_splits;
  const int begin = lo + split * per_split;
  const int end = (begin + per_split < p + 1) ? begin + per_split : p + 1;
  const int32_t* table = block_table + static_cast<int64_t>(req_of_token[t]) * max_blocks;
  const int64_t head_stride = static_cast<int64_t>(d) << bs_shift;   // pages hold a power of two of tokens
  float* lds_o = lds + wave * kpi * d;
  float* state = lds + NW * kpi * d;      // [NW][GC][d + 2]
  const int h0 = (blockIdx.y % chunks) * GC;

  uint32_t qp[GC][8];
#pragma unroll
  for (int i = 0; i < GC; ++i) {
    const int h = hk * group + ((h0 + i < group) ? h0 + i : h0);
    const uint4* src = reinterpret_cast<const uint4*>(q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * d + part * 16);
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    if (active) { a = src[0]; b = src[1]; }
    qp[i][0] = a.x; qp[i][1] = a.y; qp[i][2] = a.z; qp[i][3] = a.w;
    qp[i][4] = b.x; qp[i][5] = b.y; qp[i][6] = b.z; qp[i][7] = b.w;
  }
  float m[GC], l[GC], o[GC][16];
#pragma unroll
  for (int i = 0; i < GC; ++i) {
    m[i] = -FLT_MAX;
    l[i] = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) o[i][c] = 0.f;
  }

  // lane x holds the page of logical block page_base + x; a round's keys lie within 64 pages of its first
  int page_base = begin >> bs_shift;
  const int last_page = p >> bs_shift;
  int my_page = (begin < end && page_base + lane <= last_page) ? table[page_base + lane] : 0;
  // keys and values of the round that starts at key j0 (every lane takes part in the page exchange)
  auto fetch = [&](int j0, KeyValue& kv) {
    if (j0 >= end) return;                                            // uniform over the wave
    if (((j0 + kpi - 1) >> bs_shift) - page_base >= 64) {             // uniform over the wave
      page_base = j0 >> bs_shift;
      my_page = (page_base + lane <= last_page) ? table[page_base + lane] : 0;
    }
    const int j = j0 + slot;
    const int64_t blk = __shfl(my_page, ((j < end ? j : j0) >> bs_shift) - page_base, 64);
    if (active && j < end) {
      const int64_t base = (blk * kv_heads + hk) * head_stride + static_cast<int64_t>(j & ((1 << bs_shift) - 1)) * d + part * 16;
      const uint4* kp = reinterpret_cast<const uint4*>(k_cache + base);
      const uint4* vp = reinterpret_cast<const uint4*>(v_cache + base);
      kv.k0 = kp[0]; kv.k1 = kp[1]; kv.v0 = vp[0]; kv.v1 = vp[1];
    }
  };

  KeyValue cur, nxt, nx2;
  cur.k0 = cur.k1 = cur.v0 = cur.v1 = make_uint4(0, 0, 0, 0);
  nxt = nx2 = cur;
  fetch(begin, cur);
  fetch(begin + kpi, nxt);
  for (int j0 = begin; j0 < end; j0 += kpi) {
    const int j = j0 + slot;
    fetch(j0 + 2 * kpi, nx2);
    const uint32_t kw[8] = {cur.k0.x, cur.k0.y, cur.k0.z, cur.k0.w, cur.k1.x, cur.k1.y, cur.k1.z, cur.k1.w};
    const uint32_t vw[8] = {cur.v0.x, cur.v0.y, cur.v0.z, cur.v0.w, cur.v1.x, cur.v1.y, cur.v1.z, cur.v1.w};
    float s[GC];
#pragma unroll
    for (int i = 0; i < GC; ++i) {
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < 8; ++c) acc = dot2(qp[i][c], kw[c], acc);
      s[i] = acc;
    }
    // add up the lanes that share the key
    if ((lpk & (lpk - 1)) == 0) {     // uniform over the launch
#pragma unroll
      for (int i = 0; i < GC; ++i) {
        if (lpk >= 2) s[i] += lane_xor1(s[i]);
        if (lpk >= 4) s[i] += lane_xor2(s[i]);
        if (lpk >= 8) s[i] += __shfl_xor(s[i], 4, 64);
        if (lpk >= 16) s[i] += lane_xor8(s[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < GC; ++i) {
        float total = 0.f;
        for (int x = 0; x < lpk; ++x) total += __shfl(s[i], slot * lpk + x, 64);
        s[i] = total;
      }
    }
    if (active && j < end) {
      float vf[16];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        vf[2 * c] = __uint_as_float(vw[c] << 16);
        vf[2 * c + 1] = __uint_as_float(vw[c] & 0xffff0000u);
      }
#pragma unroll
      for (int i = 0; i < GC; ++i) {
        const float sc = s[i] * scale;
        if (sc > m[i]) {  // a new maximum: bring what was gathered so far to its scale
          const float corr = __expf(m[i] - sc);
          l[i] *= corr;
#pragma unroll
          for (int c = 0; c < 16; ++c) o[i][c] *= corr;
          m[i] = sc;
        }
        const float w = __expf(sc - m[i]);
        l[i] += w;
#pragma unroll
        for (int c = 0; c < 16; ++c) o[i][c] += w * vf[c];
      }
    }
    cur = nxt;
    nxt = nx2;
  }

  // The lane groups' states are combined: the maximum over all groups, every group's
  // weight exp(m - max), the sum of weights by a fixed butterfly, and the weighted
  // value sums through LDS, added in group order. The wave's state goes to `state`.
#pragma unroll
  for (int i = 0; i < GC; ++i) {
    if (h0 + i >= group) break;   // uniform over the block
    const float big = wave_max(m[i]);
    const float e = __expf(m[i] - big);   // 0 for groups that saw no key
    const float total = wave_sum((active && part == 0) ? l[i] * e : 0.f);
    wave_lds_sync();              // the previous head's sums have been read (the room is this wave's own)
    if (active) {
      float4* dst = reinterpret_cast<float4*>(lds_o + slot * d + part * 16);
      dst[0] = make_float4(o[i][0] * e, o[i][1] * e, o[i][2] * e, o[i][3] * e);
      dst[1] = make_float4(o[i][4] * e, o[i][5] * e, o[i][6] * e, o[i][7] * e);
      dst[2] = make_float4(o[i][8] * e, o[i][9] * e, o[i][10] * e, o[i][11] * e);
      dst[3] = make_float4(o[i][12] * e, o[i][13] * e, o[i][14] * e, o[i][15] * e);
    }
    wave_lds_sync();
    float* mine = state + (wave * GC + i) * (d + 2);
    for (int c = lane; c < d; c += 64) {
      float acc = 0.f;
#pragma unroll 8
      for (int s2 = 0; s2 < kpi; ++s2) acc += lds_o[s2 * d + c];
      mine[2 + c] = acc;
    }
    if (lane == 0) { mine[0] = big; mine[1] = total; }
  }
  __syncthreads();

  // the waves' states are combined in wave order; thread x takes channel x % d of head x / d
  for (int x = threadIdx.x; x < GC * d; x += 64 * NW) {
    const int i = x / d, c = x % d;
    if (h0 + i >= group) break;
    const int h = hk * group + h0 + i;
    const float* st = state + i * (d + 2);
    float big = st[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) big = fmaxf(big, st[w * GC * (d + 2)]);
    float total = 0.f, acc = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float e = __expf(st[w * GC * (d + 2)] - big);
      total += st[w * GC * (d + 2) + 1] * e;
      acc += st[w * GC * (d + 2) + 2 + c] * e;
    }
    if (n_parts == 1) {
      store_f32(out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * d + c, acc / total);
    } else {
      float* dst = partial + ((static_cast<int64_t>(blockIdx.x) * heads + h) * n_parts + blockIdx.z) * (d + 2);
      dst[2 + c] = acc;
      if (c == 0) { dst[0] = big; dst[1] = total; }
    }
  }
}

// Combines the splits' states of one (token, head) in split order.
__global__ void __launch_bounds__(64) attention_merge_kernel(bf16_t* __restrict__ out, int64_t out_stride,
                                                             const float* __restrict__ partial,
                                                             const int32_t* __restrict__ rows, int heads, int d,
                                                             int n_splits) {
  const int t = rows ? rows[blockIdx.x] : blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* src = partial + (static_cast<int64_t>(blockIdx.x) * heads + h) * n_splits * (d + 2);
  // lane s holds split s's maximum and sum (n_splits <= 64)
  const float m = lane < n_splits ? src[lane * (d + 2)] : -FLT_MAX;
  const float l = lane < n_splits ? src[lane * (d + 2) + 1] : 0.f;
  const float big = wave_max(m);
  const float e = __expf(m - big);
  const float total = wave_sum(l * e);
  // every lane takes part in every round, so that the weights can be read from all 64 lanes
  for (int c0 = 0; c0 < d; c0 += 64) {
    const int c = c0 + lane;
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < n_splits; ++s) {
      const float w = __shfl(e, s, 64);
      if (c < d) acc += src[s * (d + 2) + 2 + c] * w;
    }
    if (c < d) store_f32(out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * d + c, acc / total);
  }
}

}  // namespace alofa

using namespace alofa;

// Waves per block: each takes a share of the keys; their states meet in LDS (which bounds their number).
extern "C" int alofa_attention_decode_waves(int d) { return d <= 128 ? 8 : 4; }

// Floats of scratch that n_splits > 1 needs.
extern "C" int64_t alofa_attention_decode_scratch(int tokens, int heads, int d, int n_splits) {
  return n_splits > 1 ? static_cast<int64_t>(tokens) * heads * n_splits * (d + 2) : 0;
}

extern "C" int alofa_attention_decode(void* out, int64_t out_stride, float* partial, const void* q, int64_t q_stride,
                                      const void* k_cache, const void* v_cache, const int32_t* block_table,
                                      int max_blocks, const int32_t* req_of_token, const int32_t* positions,
                                      const int32_t* rows, int tokens, int heads, int kv_heads, int d, int block_size, int window,
                                      float scale, int n_splits, hipStream_t stream) {
  ALOFA_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
                "attention_decode: tokens=%d heads=%d kv_heads=%d (kv_heads must divide heads)", tokens, heads, kv_heads);
  ALOFA_REQUIRE(d >= 16 && d <= 256 && d % 16 == 0, "attention_decode: head size %d must be 16..256 in steps of 16", d);
  ALOFA_REQUIRE(block_size > 0 && (block_size & (block_size - 1)) == 0 && max_blocks > 0 && window >= 0,
                "attention_decode: block_size=%d must be a power of two; max_blocks=%d window=%d", block_size, max_blocks, window);
  int bs_shift = 0;
  while ((1 << bs_shift) < block_size) ++bs_shift;
  ALOFA_REQUIRE(n_splits >= 1 && n_splits <= kMaxSplits && (n_splits == 1 || partial), "attention_decode: n_splits=%d (1..%d) needs scratch when above 1", n_splits, kMaxSplits);
  ALOFA_REQUIRE(q_stride % 8 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0, "attention_decode: q rows must be 16-byte aligned");
  const int group = heads / kv_heads;
  const int kpi = 64 / (d / 16);
  const int gc = group == 1 ? 1 : group == 2 ? 2 : group == 3 ? 3 : 4;
  const int nw = alofa_attention_decode_waves(d);
  dim3 grid(tokens, kv_heads * ((group + gc - 1) / gc), n_splits);
  const size_t lds = (static_cast<size_t>(nw) * kpi * d + static_cast<size_t>(nw) * gc * (d + 2)) * sizeof(float);
#define ALOFA_DECODE(GC, NW)                                                                                              \
  attention_decode_kernel<GC, NW><<<grid, 64 * NW, lds, stream>>>(                                                        \
      static_cast<bf16_t*>(out), out_stride, partial, static_cast<const bf16_t*>(q), q_stride,                            \
      static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), block_table, max_blocks, req_of_token,    \
      positions, rows, heads, kv_heads, d, bs_shift, window, scale)
  if (nw == 8) {
    if (gc == 1) ALOFA_DECODE(1, 8);
    else if (gc == 2) ALOFA_DECODE(2, 8);
    else if (gc == 3) ALOFA_DECODE(3, 8);
    else ALOFA_DECODE(4, 8);
  } else {
    if (gc == 1) ALOFA_DECODE(1, 4);
    else if (gc == 2) ALOFA_DECODE(2, 4);
    else if (gc == 3) ALOFA_DECODE(3, 4);
    else ALOFA_DECODE(4, 4);
  }
#undef ALOFA_DECODE
  if (check_launch("attention_decode")) return 1;
  if (n_splits > 1) {
    attention_merge_kernel<<<dim3(tokens, heads), 64, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, partial, rows, heads, d, n_splits);
    return check_launch("attention_merge");
  }
  return 0;
}
