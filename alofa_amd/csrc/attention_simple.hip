// Paged causal grouped-query attention, the always-valid kernel: one wavefront
// per (token, query head). Query token t of request r stands at absolute
// position p = positions[t] and sees the keys lo..p of r's pages, lo = 0 or
// p - window + 1. Key head = query head / (heads / kv_heads).
//
// Arithmetic of a plain loop: the dot product is accumulated in Acc and rounded
// to float, then multiplied by the float scale; the maximum and exp are float;
// the sum of the weights and the weighted sum of the values are accumulated in
// Acc in ascending key order per channel, and divided once at the end. The
// order depends only on the key's position, so a row's result is the same
// however the tokens were cut into steps and whichever pages hold them.
// Cache layout: keys [block, kv_head, slot_in_block, d], values transposed [block, kv_head, d, slot_in_block].
#include "common.h"

#include <float.h>

namespace alofa {

constexpr int kMaxHeadDim = 256;

template <typename T, typename Acc>
__device__ __forceinline__ float score_of(const float* qs, const T* __restrict__ k_cache,
                                          const int32_t* __restrict__ table, int j, int hk, int kv_heads, int d,
                                          int block_size, float scale) {
  const int64_t blk = table[j / block_size];
  const T* k = k_cache + ((blk * kv_heads + hk) * block_size + (j % block_size)) * static_cast<int64_t>(d);
  Acc acc = 0;
  for (int c = 0; c < d; ++c) acc += static_cast<Acc>(qs[c]) * static_cast<Acc>(load_f32(k + c));
  return static_cast<float>(acc) * scale;
}

template <typename T, typename Acc>
__global__ void __launch_bounds__(64) attention_simple_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int32_t* __restrict__ block_table,
    int max_blocks, const int32_t* __restrict__ req_of_token, const int32_t* __restrict__ positions, int heads,
    int kv_heads, int d, int block_size, int window, float scale) {
  __shared__ float qs[kMaxHeadDim];
  __shared__ float es[kWave];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int hk = h / (heads / kv_heads);
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int32_t* table = block_table + static_cast<int64_t>(req_of_token[t]) * max_blocks;
  const T* qrow = q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * d;
  for (int c = lane; c < d; c += kWave) qs[c] = load_f32(qrow + c);
  __syncthreads();

  float m = -FLT_MAX;
  for (int j = lo + lane; j <= p; j += kWave)
    m = fmaxf(m, score_of<T, Acc>(qs, k_cache, table, j, hk, kv_heads, d, block_size, scale));
  m = wave_max(m);

  Acc z = 0;
  Acc o[kMaxHeadDim / kWave];
#pragma unroll
  for (int i = 0; i < kMaxHeadDim / kWave; ++i) o[i] = 0;
  for (int j0 = lo; j0 <= p; j0 += kWave) {
    const int j = j0 + lane;
    es[lane] = (j <= p) ? expf(score_of<T, Acc>(qs, k_cache, table, j, hk, kv_heads, d, block_size, scale) - m) : 0.f;
    __syncthreads();
    const int n = (p - j0 + 1 < kWave) ? p - j0 + 1 : kWave;
    for (int jj = 0; jj < n; ++jj) {
      const Acc e = static_cast<Acc>(es[jj]);
      z += e;
      const int jk = j0 + jj;
      const int64_t blk = table[jk / block_size];
      const T* v = v_cache + (blk * kv_heads + hk) * static_cast<int64_t>(d) * block_size + (jk % block_size);
#pragma unroll
      for (int i = 0; i < kMaxHeadDim / kWave; ++i) {
        const int c = lane + i * kWave;
        if (c < d) o[i] += e * static_cast<Acc>(load_f32(v + static_cast<int64_t>(c) * block_size));
      }
    }
    __syncthreads();
  }
  T* orow = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * d;
#pragma unroll
  for (int i = 0; i < kMaxHeadDim / kWave; ++i) {
    const int c = lane + i * kWave;
    if (c < d) store_f32(orow + c, static_cast<float>(o[i] / z));
  }
}

}  // namespace alofa

using namespace alofa;

extern "C" int alofa_attention_simple(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                      const void* k_cache, const void* v_cache, int dtype,
                                      const int32_t* block_table, int max_blocks, const int32_t* req_of_token,
                                      const int32_t* positions, int tokens, int heads, int kv_heads, int d,
                                      int block_size, int window, float scale, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
                "attention: tokens=%d heads=%d kv_heads=%d (kv_heads must divide heads)", tokens, heads, kv_heads);
  ALOFA_REQUIRE(d > 0 && d <= kMaxHeadDim, "attention: head size %d is outside 1..%d", d, kMaxHeadDim);
  ALOFA_REQUIRE(block_size > 0 && max_blocks > 0 && window >= 0, "attention: block_size=%d max_blocks=%d window=%d", block_size, max_blocks, window);
  dim3 grid(tokens, heads);
  if (dtype == kF32 && exact)
    attention_simple_kernel<float, double><<<grid, 64, 0, stream>>>(
        static_cast<float*>(out), out_stride, static_cast<const float*>(q), q_stride, static_cast<const float*>(k_cache),
        static_cast<const float*>(v_cache), block_table, max_blocks, req_of_token, positions, heads, kv_heads, d, block_size, window, scale);
  else if (dtype == kF32)
    attention_simple_kernel<float, float><<<grid, 64, 0, stream>>>(
        static_cast<float*>(out), out_stride, static_cast<const float*>(q), q_stride, static_cast<const float*>(k_cache),
        static_cast<const float*>(v_cache), block_table, max_blocks, req_of_token, positions, heads, kv_heads, d, block_size, window, scale);
  else if (dtype == kBF16 && !exact)
    attention_simple_kernel<bf16_t, float><<<grid, 64, 0, stream>>>(
        static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(k_cache),
        static_cast<const bf16_t*>(v_cache), block_table, max_blocks, req_of_token, positions, heads, kv_heads, d, block_size, window, scale);
  else
    ALOFA_REQUIRE(false, "attention: unsupported dtype %d with exact=%d", dtype, exact);
  return check_launch("attention_simple");
}
