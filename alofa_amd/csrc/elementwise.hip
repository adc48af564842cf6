// Row-wise and element-wise kernels: embedding gather, RMSNorm (with an
// optional row gather), rotary positions fused with the cache write, SwiGLU.
//
// "exact" variants (Acc = double) keep the arithmetic of a float32 model with
// float64 accumulators and one rounding where a plain implementation rounds;
// the others accumulate in float.
#include "common.h"

namespace alofa {

// ---- embedding -------------------------------------------------------------
// hidden[t, :] = table[ids[t], :], widened to float. No scaling.
template <typename TW>
__global__ void embed_gather_kernel(float* __restrict__ out, const TW* __restrict__ table,
                                    const int32_t* __restrict__ ids, int width) {
  const int t = blockIdx.x;
  const TW* row = table + static_cast<int64_t>(ids[t]) * width;
  float* dst = out + static_cast<int64_t>(t) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = load_f32(row + c);
}

// ---- RMSNorm ---------------------------------------------------------------
// y = x * 1/sqrt(mean(x^2) + eps) * w per row; row r of the output is made from
// row rows[r] of x when `rows` is given. x is the float residual stream.
template <typename TO, typename Acc>
__global__ void __launch_bounds__(256) rmsnorm_kernel(TO* __restrict__ out, const float* __restrict__ x,
                                                      const float* __restrict__ w,
                                                      const int32_t* __restrict__ rows, int width, float eps) {
  __shared__ Acc scratch[4];
  const int r = blockIdx.x;
  const float* src = x + static_cast<int64_t>(rows ? rows[r] : r) * width;
  TO* dst = out + static_cast<int64_t>(r) * width;
  // rows of up to 256 * kKeep values stay in registers between the two passes, and their weights are on
  // their way while the squares are summed; wider rows are read twice
  constexpr int kKeep = 8;
  if (width <= 256 * kKeep) {
    float xs[kKeep], ws[kKeep];
    Acc ss = 0;
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
      const int c = threadIdx.x + 256 * i;
      xs[i] = c < width ? src[c] : 0.f;
      ws[i] = c < width ? w[c] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {      // ascending c, as the strided loop below
      const Acc v = static_cast<Acc>(xs[i]);
      ss += v * v;
    }
    ss = block_sum<Acc, 256>(ss, scratch);
    const Acc scale = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(width) + static_cast<Acc>(eps));
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
      const int c = threadIdx.x + 256 * i;
      if (c < width) store_f32(dst + c, static_cast<float>(static_cast<Acc>(xs[i]) * scale * static_cast<Acc>(ws[i])));
    }
    return;
  }
  Acc ss = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    Acc v = static_cast<Acc>(src[c]);
    ss += v * v;
  }
  ss = block_sum<Acc, 256>(ss, scratch);
  const Acc scale = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(width) + static_cast<Acc>(eps));
  for (int c = threadIdx.x; c < width; c += 256)
    store_f32(dst + c, static_cast<float>(static_cast<Acc>(src[c]) * scale * static_cast<Acc>(w[c])));
}

// ---- rotary positions + cache write ----------------------------------------
// qkv holds, per token, the query heads, then the key heads, then the value
// heads. Queries and keys are rotated by the token's absolute position with the
// half-split pairing (j, j + d/2); queries are rotated in place, rotated keys
// and plain values go to the token's cache slot. Products and the sum are
// separate float operations (no fused multiply-add), as in a plain loop.
// Cache layout: keys [block, kv_head, slot_in_block, d], values transposed [block, kv_head, d, slot_in_block]
// (consecutive keys of one channel are contiguous: the order in which the matrix cores reduce over keys).
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t, const int32_t* __restrict__ positions,
                                     const int64_t* __restrict__ slots, T* __restrict__ k_cache,
                                     T* __restrict__ v_cache, int heads, int kv_heads, int d, int block_size,
                                     int write_cache) {
#pragma clang fp contract(off)
  const int t = blockIdx.x;
  const int half = d / 2;
  T* row = qkv + static_cast<int64_t>(t) * row_stride;
  const int pos = positions[t];
  const float* cs = cos_t + static_cast<int64_t>(pos) * half;
  const float* sn = sin_t + static_cast<int64_t>(pos) * half;
  const int64_t slot = slots ? slots[t] : 0;
  const int64_t blk = slot / block_size, off = slot % block_size;
  const int rot_pairs = (heads + kv_heads) * half;
  for (int i = threadIdx.x; i < rot_pairs; i += blockDim.x) {
    const int head = i / half, j = i % half;
    T* x = row + static_cast<int64_t>(head) * d;
    const float a = load_f32(x + j), b = load_f32(x + j + half);
    const float c = cs[j], s = sn[j];
    const float lo = a * c - b * s;
    const float hi = b * c + a * s;
    if (head < heads) {
      store_f32(x + j, lo);
      store_f32(x + j + half, hi);
    } else if (write_cache) {
      const int hk = head - heads;
      T* dst = k_cache + ((blk * kv_heads + hk) * block_size + off) * d;
      store_f32(dst + j, lo);
      store_f32(dst + j + half, hi);
    }
  }
  if (write_cache) {
    const T* v = row + static_cast<int64_t>(heads + kv_heads) * d;
    for (int i = threadIdx.x; i < kv_heads * d; i += blockDim.x) {
      const int hk = i / d, c = i % d;
      v_cache[((blk * kv_heads + hk) * d + c) * block_size + off] = v[i];      // values lie transposed: [channel][slot]
    }
  }
}

// ---- SwiGLU (unfused) ------------------------------------------------------
// out = gate / (1 + exp(-gate)) * up, element-wise.
template <typename T, typename Acc>
__global__ void swiglu_kernel(T* __restrict__ out, const T* __restrict__ gate, const T* __restrict__ up, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const Acc g = static_cast<Acc>(load_f32(gate + i));
  const Acc u = static_cast<Acc>(load_f32(up + i));
  store_f32(out + i, static_cast<float>(g / (static_cast<Acc>(1) + exp(-g)) * u));
}

}  // namespace alofa

using namespace alofa;

extern "C" int alofa_embed_gather(float* out, const void* table, int table_dtype, const int32_t* ids, int tokens,
                                  int width, hipStream_t stream) {
  ALOFA_REQUIRE(tokens > 0 && width > 0, "embed_gather: tokens=%d width=%d must be positive", tokens, width);
  const int threads = width >= 256 ? 256 : 64;
  if (table_dtype == kF32)
    embed_gather_kernel<float><<<tokens, threads, 0, stream>>>(out, static_cast<const float*>(table), ids, width);
  else if (table_dtype == kBF16)
    embed_gather_kernel<bf16_t><<<tokens, threads, 0, stream>>>(out, static_cast<const bf16_t*>(table), ids, width);
  else
    ALOFA_REQUIRE(false, "embed_gather: unknown table dtype %d", table_dtype);
  return check_launch("embed_gather");
}

extern "C" int alofa_rmsnorm(void* out, int out_dtype, const float* x, const float* w, const int32_t* rows,
                             int n_rows, int width, float eps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n_rows > 0 && width > 0, "rmsnorm: rows=%d width=%d must be positive", n_rows, width);
  if (out_dtype == kF32 && exact)
    rmsnorm_kernel<float, double><<<n_rows, 256, 0, stream>>>(static_cast<float*>(out), x, w, rows, width, eps);
  else if (out_dtype == kF32)
    rmsnorm_kernel<float, float><<<n_rows, 256, 0, stream>>>(static_cast<float*>(out), x, w, rows, width, eps);
  else if (out_dtype == kBF16 && !exact)
    rmsnorm_kernel<bf16_t, float><<<n_rows, 256, 0, stream>>>(static_cast<bf16_t*>(out), x, w, rows, width, eps);
  else
    ALOFA_REQUIRE(false, "rmsnorm: unsupported out dtype %d with exact=%d", out_dtype, exact);
  return check_launch("rmsnorm");
}

extern "C" int alofa_rope_kv_write(void* qkv, int dtype, int64_t row_stride, const float* cos_t, const float* sin_t,
                                   const int32_t* positions, const int64_t* slots, void* k_cache, void* v_cache,
                                   int tokens, int heads, int kv_heads, int d, int block_size, int write_cache,
                                   hipStream_t stream) {
  ALOFA_REQUIRE(tokens > 0 && heads > 0 && kv_heads >= 0, "rope_kv_write: tokens=%d heads=%d kv_heads=%d", tokens, heads, kv_heads);
  ALOFA_REQUIRE(d > 0 && d % 2 == 0, "rope_kv_write: head size %d must be positive and even", d);
  ALOFA_REQUIRE(!write_cache || (slots && k_cache && v_cache && block_size > 0), "rope_kv_write: cache write needs slots, caches and a block size");
  const int threads = 256;
  if (dtype == kF32)
    rope_kv_write_kernel<float><<<tokens, threads, 0, stream>>>(static_cast<float*>(qkv), row_stride, cos_t, sin_t, positions, slots,
                                                                 static_cast<float*>(k_cache), static_cast<float*>(v_cache), heads,
                                                                 kv_heads, d, block_size, write_cache);
  else if (dtype == kBF16)
    rope_kv_write_kernel<bf16_t><<<tokens, threads, 0, stream>>>(static_cast<bf16_t*>(qkv), row_stride, cos_t, sin_t, positions, slots,
                                                                  static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), heads,
                                                                  kv_heads, d, block_size, write_cache);
  else
    ALOFA_REQUIRE(false, "rope_kv_write: unknown dtype %d", dtype);
  return check_launch("rope_kv_write");
}

extern "C" int alofa_swiglu(void* out, const void* gate, const void* up, int dtype, int64_t n, int exact,
                            hipStream_t stream) {
  ALOFA_REQUIRE(n > 0, "swiglu: n=%lld must be positive", static_cast<long long>(n));
  const int threads = 256;
  const int blocks = static_cast<int>((n + threads - 1) / threads);
  if (dtype == kF32 && exact)
    swiglu_kernel<float, double><<<blocks, threads, 0, stream>>>(static_cast<float*>(out), static_cast<const float*>(gate), static_cast<const float*>(up), n);
  else if (dtype == kF32)
    swiglu_kernel<float, float><<<blocks, threads, 0, stream>>>(static_cast<float*>(out), static_cast<const float*>(gate), static_cast<const float*>(up), n);
  else if (dtype == kBF16)
    swiglu_kernel<bf16_t, float><<<blocks, threads, 0, stream>>>(static_cast<bf16_t*>(out), static_cast<const bf16_t*>(gate), static_cast<const bf16_t*>(up), n);
  else
    ALOFA_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
  return check_launch("swiglu");
}
