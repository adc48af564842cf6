// Row-wise and element-wise kernels: embedding gather, RMSNorm (with an
// optional row gather), rotary positions fused with the cache write, SwiGLU.
//
// "exact" variants (Acc = double) keep the arithmetic of a float32 model with
// float64 accumulators and one rounding where a plain implementation rounds;
// the others accumulate in float.
#include "common.h"

namespace alofa {

// ---- embedding -------------------------------------------------------------
// hidden[t, :] = table[ids[t], :], widened to float. No scaling. An id below zero stands for a token
// that never left the device: -(s + 1) means store[s], where the choice of the last step put the
// token of request slot s (brought into the vocabulary, so that no table row outside it is read).
template <typename TW>
__global__ void embed_gather_kernel(float* __restrict__ out, const TW* __restrict__ table,
                                    const int32_t* __restrict__ ids, int width, const int32_t* __restrict__ store, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0) {
    id = store[-(id + 1)];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  }
  const TW* row = table + static_cast<int64_t>(id) * width;
  float* dst = out + static_cast<int64_t>(t) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = load_f32(row + c);
}

// ---- RMSNorm ---------------------------------------------------------------
// y = x * 1/sqrt(mean(x^2) + eps) * w per row; row r of the output is made from
// row rows[r] of x when `rows` is given. x is the float residual stream.
// K4 > 0: the row (a multiple of four wide, at most 1,024 K4 values, 16-byte aligned) stays in registers as K4
// groups of four per thread between the sum of its squares and the scaling, and its weights are on their way
// meanwhile; K4 = 0: any row, read twice.
template <typename TO, typename Acc, int K4>
__global__ void __launch_bounds__(256) rmsnorm_kernel(TO* __restrict__ out, const float* __restrict__ x,
                                                      const float* __restrict__ w,
                                                      const int32_t* __restrict__ rows, int width, float eps) {
  __shared__ Acc scratch[4];
  const int r = blockIdx.x;
  const float* src = x + static_cast<int64_t>(rows ? rows[r] : r) * width;
  TO* dst = out + static_cast<int64_t>(r) * width;
  if constexpr (K4 > 0) {
    float4 xs[K4], ws[K4];
    const int groups = width / 4;
#pragma unroll
    for (int i = 0; i < K4; ++i) {
      const int g = threadIdx.x + 256 * i;
      xs[i] = g < groups ? reinterpret_cast<const float4*>(src)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
      ws[i] = g < groups ? reinterpret_cast<const float4*>(w)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    Acc ss = 0;
#pragma unroll
    for (int i = 0; i < K4; ++i) {      // ascending columns within the thread
      const Acc a = static_cast<Acc>(xs[i].x), b = static_cast<Acc>(xs[i].y), c = static_cast<Acc>(xs[i].z), d = static_cast<Acc>(xs[i].w);
      ss += a * a;
      ss += b * b;
      ss += c * c;
      ss += d * d;
    }
    ss = block_sum<Acc, 256>(ss, scratch);
    const Acc scale = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(width) + static_cast<Acc>(eps));
#pragma unroll
    for (int i = 0; i < K4; ++i) {
      const int g = threadIdx.x + 256 * i;
      if (g < groups) {
        store_f32(dst + 4 * g + 0, static_cast<float>(static_cast<Acc>(xs[i].x) * scale * static_cast<Acc>(ws[i].x)));
        store_f32(dst + 4 * g + 1, static_cast<float>(static_cast<Acc>(xs[i].y) * scale * static_cast<Acc>(ws[i].y)));
        store_f32(dst + 4 * g + 2, static_cast<float>(static_cast<Acc>(xs[i].z) * scale * static_cast<Acc>(ws[i].z)));
        store_f32(dst + 4 * g + 3, static_cast<float>(static_cast<Acc>(xs[i].w) * scale * static_cast<Acc>(ws[i].w)));
      }
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

// The same for bfloat16 and head sizes in steps of 16. Rotation: eight pairs per thread with 16-byte accesses;
// the arithmetic and the rounding are those of the kernel above, element for element. Values: a thread takes one
// channel of eight consecutive tokens; where these lie in eight consecutive, aligned slots of one page (portions
// of prompts do) they leave as one 16-byte store into the transposed cache instead of eight scattered ones.
__global__ void __launch_bounds__(256) rope_kv_write_vec_kernel(
    bf16_t* __restrict__ qkv, int64_t row_stride, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int32_t* __restrict__ positions, const int64_t* __restrict__ slots, bf16_t* __restrict__ k_cache,
    bf16_t* __restrict__ v_cache, int tokens, int heads, int kv_heads, int d, int block_size, int write_cache) {
#pragma clang fp contract(off)
  const int half = d / 2;
  const int rot_units = (heads + kv_heads) * (half / 8);
  const int64_t rot_threads = static_cast<int64_t>(tokens) * rot_units;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx < rot_threads) {
    const int t = static_cast<int>(idx / rot_units), u = static_cast<int>(idx % rot_units);
    bf16_t* row = qkv + static_cast<int64_t>(t) * row_stride;
    const int head = u / (half / 8), j = (u % (half / 8)) * 8;
    const int pos = positions[t];
    const float* cs = cos_t + static_cast<int64_t>(pos) * half + j;
    const float* sn = sin_t + static_cast<int64_t>(pos) * half + j;
    bf16_t* x = row + static_cast<int64_t>(head) * d + j;
    const uint4 av = *reinterpret_cast<const uint4*>(x), bv = *reinterpret_cast<const uint4*>(x + half);
    const float4 c0 = *reinterpret_cast<const float4*>(cs), c1 = *reinterpret_cast<const float4*>(cs + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(sn), s1 = *reinterpret_cast<const float4*>(sn + 4);
    const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
    const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w}, sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // two elements per 32-bit word, the lower one first
      const float a0 = __uint_as_float(aw[e] << 16), a1 = __uint_as_float(aw[e] & 0xffff0000u);
      const float b0 = __uint_as_float(bw[e] << 16), b1 = __uint_as_float(bw[e] & 0xffff0000u);
      lo[e] = pack_bf16x2(a0 * c[2 * e] - b0 * sv[2 * e], a1 * c[2 * e + 1] - b1 * sv[2 * e + 1]);
      hi[e] = pack_bf16x2(b0 * c[2 * e] + a0 * sv[2 * e], b1 * c[2 * e + 1] + a1 * sv[2 * e + 1]);
    }
    bf16_t* dst = x;
    if (head >= heads) {
      if (!write_cache) return;
      const int64_t slot = slots[t];
      dst = k_cache + ((slot / block_size * kv_heads + (head - heads)) * block_size + slot % block_size) * d + j;
    }
    *reinterpret_cast<uint4*>(dst) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    *reinterpret_cast<uint4*>(dst + half) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    return;
  }
  if (!write_cache) return;
  // values: thread = (group of eight tokens, key head, channel); consecutive lanes take consecutive channels
  const int64_t v_idx = idx - rot_threads;
  const int per_group = kv_heads * d;
  const int64_t group = v_idx / per_group;
  if (group * 8 >= tokens) return;
  const int hk = static_cast<int>(v_idx % per_group) / d, ch = static_cast<int>(v_idx % per_group) % d;
  const int t0 = static_cast<int>(group) * 8, n = (tokens - t0 < 8) ? tokens - t0 : 8;
  int64_t slot[8];
  uint32_t val[8];
  bool run = n == 8 && block_size % 8 == 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int t = t0 + (e < n ? e : 0);
    slot[e] = slots[t];
    val[e] = qkv[static_cast<int64_t>(t) * row_stride + static_cast<int64_t>(heads + kv_heads + hk) * d + ch];
    run = run && slot[e] == slot[0] + e;
  }
  run = run && slot[0] % 8 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0;
  if (run) {      // eight slots of one page side by side (pages hold a multiple of eight tokens)
    bf16_t* dst = v_cache + ((slot[0] / block_size * kv_heads + hk) * d + ch) * block_size + slot[0] % block_size;
    *reinterpret_cast<uint4*>(dst) = make_uint4(val[0] | (val[1] << 16), val[2] | (val[3] << 16), val[4] | (val[5] << 16), val[6] | (val[7] << 16));
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (e < n) v_cache[((slot[e] / block_size * kv_heads + hk) * d + ch) * block_size + slot[e] % block_size] = static_cast<bf16_t>(val[e]);
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

// store: null when every id is a token (the caller has checked them against the vocabulary); else ids below
// zero name slots of `store` (the caller has checked them against its length)
extern "C" int alofa_embed_gather(float* out, const void* table, int table_dtype, const int32_t* ids, int tokens,
                                  int width, const int32_t* store, int vocab, hipStream_t stream) {
  ALOFA_REQUIRE(tokens > 0 && width > 0 && vocab > 0, "embed_gather: tokens=%d width=%d vocab=%d must be positive", tokens, width, vocab);
  const int threads = width >= 256 ? 256 : 64;
  if (table_dtype == kF32)
    embed_gather_kernel<float><<<tokens, threads, 0, stream>>>(out, static_cast<const float*>(table), ids, width, store, vocab);
  else if (table_dtype == kBF16)
    embed_gather_kernel<bf16_t><<<tokens, threads, 0, stream>>>(out, static_cast<const bf16_t*>(table), ids, width, store, vocab);
  else
    ALOFA_REQUIRE(false, "embed_gather: unknown table dtype %d", table_dtype);
  return check_launch("embed_gather");
}

extern "C" int alofa_rmsnorm(void* out, int out_dtype, const float* x, const float* w, const int32_t* rows,
                             int n_rows, int width, float eps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n_rows > 0 && width > 0, "rmsnorm: rows=%d width=%d must be positive", n_rows, width);
  // rows that stay in registers: up to 8,192 wide, a multiple of four, 16-byte aligned (x rows, w and width * 4 bytes)
  const bool vec = width % 4 == 0 && width <= 8192 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
  const int k4 = !vec ? 0 : width <= 1024 ? 1 : width <= 2048 ? 2 : width <= 4096 ? 4 : 8;
#define ALOFA_RMSNORM(TO, ACC)                                                                                                   \
  switch (k4) {                                                                                                                   \
    case 1: rmsnorm_kernel<TO, ACC, 1><<<n_rows, 256, 0, stream>>>(static_cast<TO*>(out), x, w, rows, width, eps); break;         \
    case 2: rmsnorm_kernel<TO, ACC, 2><<<n_rows, 256, 0, stream>>>(static_cast<TO*>(out), x, w, rows, width, eps); break;         \
    case 4: rmsnorm_kernel<TO, ACC, 4><<<n_rows, 256, 0, stream>>>(static_cast<TO*>(out), x, w, rows, width, eps); break;         \
    case 8: rmsnorm_kernel<TO, ACC, 8><<<n_rows, 256, 0, stream>>>(static_cast<TO*>(out), x, w, rows, width, eps); break;         \
    default: rmsnorm_kernel<TO, ACC, 0><<<n_rows, 256, 0, stream>>>(static_cast<TO*>(out), x, w, rows, width, eps);               \
  }
  if (out_dtype == kF32 && exact) {
    ALOFA_RMSNORM(float, double)
  } else if (out_dtype == kF32) {
    ALOFA_RMSNORM(float, float)
  } else if (out_dtype == kBF16 && !exact) {
    ALOFA_RMSNORM(bf16_t, float)
  } else {
    ALOFA_REQUIRE(false, "rmsnorm: unsupported out dtype %d with exact=%d", out_dtype, exact);
  }
#undef ALOFA_RMSNORM
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
  else if (dtype == kBF16 && d % 16 == 0 && row_stride % 8 == 0 && reinterpret_cast<uintptr_t>(qkv) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(cos_t) % 16 == 0 && reinterpret_cast<uintptr_t>(sin_t) % 16 == 0 &&
           (!write_cache || reinterpret_cast<uintptr_t>(k_cache) % 16 == 0)) {
    const int64_t threads_needed = static_cast<int64_t>(tokens) * (heads + kv_heads) * (d / 16) +
                                   (write_cache ? static_cast<int64_t>((tokens + 7) / 8) * kv_heads * d : 0);
    const int64_t blocks = (threads_needed + 255) / 256;
    rope_kv_write_vec_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
        static_cast<bf16_t*>(qkv), row_stride, cos_t, sin_t, positions, slots, static_cast<bf16_t*>(k_cache),
        static_cast<bf16_t*>(v_cache), tokens, heads, kv_heads, d, block_size, write_cache);
  } else if (dtype == kBF16)
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
