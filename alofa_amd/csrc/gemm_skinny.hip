// Matrix products for few rows (decode steps and small portions), bfloat16:
// out[m, n] = sum_k A[m, k] * W[n, k] with M <= 64. The work is streaming W
// once from memory; the arithmetic rides on MFMA 16x16x32 tiles.
//
// A block of kWaves wavefronts owns 16 * NT output columns. The waves split K
// among themselves in interleaved steps of 32 (so that together they read
// contiguous runs of every weight row), each accumulates its share for all
// rows in registers, and the partial sums meet in LDS, added in wave order:
// the result is the same on every run and for every batch the row is part of
// (M only selects how many 16-row tiles are computed).
//
// With few output columns the blocks are too few to pull the weights at speed,
// so K is also split across blocks (blockIdx.y): every block leaves its partial
// tiles in a workspace and bumps a counter of its column tile; the block that
// arrives last adds the partial tiles in split order (not in arrival order, so
// the sum is the same on every run), runs the epilogue and puts the counter
// back to zero. Nobody waits for anybody. The workspace is uncached device
// memory (common.h): a block's partial tiles are in memory once its stores have
// been acknowledged, which every wave waits for before the block is counted.
//
// With kNorm the rows of A are the float residual stream and the kernel applies an RMSNorm on the
// way: a fragment is x * w_norm rounded to bfloat16, the sum of squares of every row is gathered
// beside the products (each block reads all of A anyway), and the row's factor 1 / sqrt(mean + eps)
// multiplies the finished sum in the epilogue. Nothing waits for the factor, so the norm costs no
// trip through memory of its own; a launch of its own it would cost as much as a small product.
//
// Operand layout of v_mfma_f32_16x16x32_bf16, lane l: A holds row l % 16,
// B holds column l % 16, both the 8 reduction indices 8 * (l / 16) .. + 7 of
// the step; D holds column l % 16, rows 4 * (l / 16) .. + 3.
#include "common.h"

#include <type_traits>

namespace alofa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

enum SkinnyEpilogue : int { kSkStore = 0, kSkResidual = 1, kSkSwiglu = 2 };


// A partial sum leaves for the workspace at device scope: written through to memory, past this
// die's L2, where blocks on every die find it.
__device__ __forceinline__ void store_partial(f32x4* p, f32x4 v) {
  float* f = reinterpret_cast<float*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) __hip_atomic_store(f + i, v[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bf16x8 load_frag(const bf16_t* __restrict__ p, bool ok) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if (ok) v = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, v);
}

// eight values of a row of A as they come from memory: bfloat16, or float with the norm's weights beside them
struct RawNormed {
  float4 lo, hi;
};
__device__ __forceinline__ void load_raw(RawNormed& dst, const void* row, int k, bool ok) {
  dst.lo = dst.hi = make_float4(0.f, 0.f, 0.f, 0.f);
  if (ok) {
    const float* p = static_cast<const float*>(row) + k;
    dst.lo = *reinterpret_cast<const float4*>(p);
    dst.hi = *reinterpret_cast<const float4*>(p + 4);
  }
}
// the sum of four squares, in one fixed order of multiply-adds (both forms of the norm below add the same numbers alike)
__device__ __forceinline__ float squares4(float4 x) {
  return __builtin_fmaf(x.w, x.w, __builtin_fmaf(x.z, x.z, __builtin_fmaf(x.y, x.y, x.x * x.x)));
}
// x * w rounded to bfloat16; the squares of x join the row's sum, four and four
__device__ __forceinline__ bf16x8 to_frag(const RawNormed& x, const RawNormed& w, float& ss) {
  ss += squares4(x.lo);
  ss += squares4(x.hi);
  const uint4 v = make_uint4(pack_bf16x2(x.lo.x * w.lo.x, x.lo.y * w.lo.y), pack_bf16x2(x.lo.z * w.lo.z, x.lo.w * w.lo.w),
                             pack_bf16x2(x.hi.x * w.hi.x, x.hi.y * w.hi.y), pack_bf16x2(x.hi.z * w.hi.z, x.hi.w * w.hi.w));
  return __builtin_bit_cast(bf16x8, v);
}

// MT: 16-row tiles of A; NT: 16-column tiles per block (kSkSwiglu: tile 0 is the
// gate matrix, tile 1 the up matrix, same columns); TO: float or bf16_t.
// kUnroll: steps of 32 along K whose loads are in flight together (twice that with the prefetch).
// kNorm: A is float [M, K] and out = epilogue(rmsnorm(A, norm_w, eps) W^T) (no split of K over blocks then).
// kNorm == 2: the same for at most eight rows. A lane's eight values of a step are then fetched by two lanes, four each
// (lane r < 8 of a row of 16 lanes the first four of row r, lane r + 8 the other four), multiplied by the norm's
// weights and rounded there, and the halves meet by a lane move: with eight rows the plain form leaves half the lanes
// of every fetch of A idle, and a fetch costs the memory pipeline the same whatever its lanes bring (gate and up
// against eight rows of 896: 8.3 against 9.3 us).
template <int MT, int NT, int kWaves, int kEpilogue, typename TO, int kUnroll, int kNorm>
__global__ void __launch_bounds__(kWaves * 64) gemm_skinny_kernel(
    TO* __restrict__ out, int64_t ldo, const void* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W,
    const bf16_t* __restrict__ W2, int64_t ldw, const float* __restrict__ bias, int M, int N, int K,
    f32x4* __restrict__ ws, int* __restrict__ counters, const float* __restrict__ norm_w, float eps, int cols) {
  __shared__ f32x4 red[kWaves][MT * NT][64];
  __shared__ float ssq[kNorm ? kWaves : 1][MT][16];
  constexpr bool kHalf = kNorm == 2;
  __shared__ int last_block;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int r = lane % 16, g = lane / 16;
  // (cols: the columns a block owns, all that its tiles hold or fewer: see launch_skinny)
  const int n0 = blockIdx.x * cols;

  const void* a_row[MT];
  bool a_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    a_ok[mt] = m < M;
    a_row[mt] = static_cast<const char*>(A) + static_cast<int64_t>(a_ok[mt] ? m : 0) * lda * (kNorm ? 4 : 2);
  }
  const bf16_t* w_row[NT];
  bool w_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = (kEpilogue == kSkSwiglu) ? n0 + r : n0 + nt * 16 + r;
    w_ok[nt] = n < N && n - n0 < cols;
    const bf16_t* base = (kEpilogue == kSkSwiglu && nt == 1) ? W2 : W;
    w_row[nt] = base + static_cast<int64_t>(w_ok[nt] ? n : 0) * ldw;
  }

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // What the epilogue adds (the bias, or the residual stream's old values) sets out now and has arrived when
  // the sums are ready: this wave finishes tiles wave, wave + kWaves, ...
  constexpr int kOutTiles = (kEpilogue == kSkSwiglu) ? MT : MT * NT;
  constexpr int kMyTiles = (kOutTiles + kWaves - 1) / kWaves;
  // With so few output tiles that they would leave most waves without work at the end (one or two), and K not
  // shared out over blocks, every thread finishes one output instead (`flat` below): thread x the x-th float of
  // the tiles as they lie in `red`. What it adds sets out now as well.
  constexpr bool kFlatTail = kOutTiles * 4 <= kWaves;
  const bool flat = kFlatTail && gridDim.y == 1;
  const int f_tile = threadIdx.x >> 8, f_r = (threadIdx.x >> 2) & 15, f_g = (threadIdx.x >> 6) & 3, f_i = threadIdx.x & 3;
  const int f_mt = (kEpilogue == kSkSwiglu) ? f_tile : f_tile / NT, f_nt = (kEpilogue == kSkSwiglu) ? 0 : f_tile % NT;
  const int f_m = f_mt * 16 + f_g * 4 + f_i, f_n = (kEpilogue == kSkSwiglu) ? n0 + f_r : n0 + f_nt * 16 + f_r;
  const bool f_ok = flat && f_tile < kOutTiles && f_m < M && f_n < N && f_n - n0 < cols;
  float f_add = 0.f;
  if (f_ok) {
    if (kEpilogue == kSkStore && bias) f_add = bias[f_n];
    if (kEpilogue == kSkResidual) f_add = load_f32(out + static_cast<int64_t>(f_m) * ldo + f_n);
  }

  float add[kMyTiles][4];
#pragma unroll
  for (int it = 0; it < kMyTiles; ++it) {
    const int tile = wave + it * kWaves;
    const int mt = (kEpilogue == kSkSwiglu) ? tile : tile / NT, nt = (kEpilogue == kSkSwiglu) ? 0 : tile % NT;
    const int n = (kEpilogue == kSkSwiglu) ? n0 + r : n0 + nt * 16 + r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = mt * 16 + g * 4 + i;
      add[it][i] = 0.f;
      if (!flat && tile < kOutTiles && n < N && n - n0 < cols && m < M) {
        if (kEpilogue == kSkStore && bias) add[it][i] = bias[n];
        if (kEpilogue == kSkResidual) add[it][i] = load_f32(out + static_cast<int64_t>(m) * ldo + n);
      }
    }
  }

  // steps of 32 along K: this block takes a contiguous share, this wave every kWaves-th step of it
  const int all_steps = (K + 31) / 32, k_splits = gridDim.y;
  const int per_split = (all_steps + k_splits - 1) / k_splits;
  const int first_step = blockIdx.y * per_split;
  const int n_steps = (first_step + per_split < all_steps) ? first_step + per_split : all_steps;
  float ss[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) ss[mt] = 0.f;
  if constexpr (!kNorm) {
    bf16x8 a_cur[kUnroll][MT], w_cur[kUnroll][NT], a_nxt[kUnroll][MT], w_nxt[kUnroll][NT];

    auto load = [&](bf16x8 (&a)[kUnroll][MT], bf16x8 (&w)[kUnroll][NT], int first) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int k = (first + u * kWaves) * 32 + g * 8;
        const bool k_ok = k < K && first + u * kWaves < n_steps;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) w[u][nt] = load_frag(w_row[nt] + k, k_ok && w_ok[nt]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a[u][mt] = load_frag(static_cast<const bf16_t*>(a_row[mt]) + k, k_ok && a_ok[mt]);
      }
    };

    load(a_cur, w_cur, first_step + wave);
    for (int s = first_step + wave; s < n_steps; s += kUnroll * kWaves) {
      if (s + kUnroll * kWaves < n_steps) load(a_nxt, w_nxt, s + kUnroll * kWaves);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_cur[u][mt], w_cur[u][nt], acc[mt][nt], 0, 0, 0);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a_cur[u][mt] = a_nxt[u][mt];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) w_cur[u][nt] = w_nxt[u][nt];
      }
    }
  } else {
    // Two sets of operands, each refilled as soon as its steps are done (no copies between sets: a copy
    // would wait for its load). Everything the first steps need sets out before anything is waited for:
    // both sets' weights and rows, then the norm's weights, which all waves share through LDS.
    static_assert(!kNorm || MT == 1, "the norm rides on products of at most 16 rows");
    extern __shared__ __attribute__((aligned(16))) float norm_lds[];      // K floats
    // (kHalf: this lane's row of A is r % 8, and of a step's eight values it fetches those from half_off on)
    const int half_off = kHalf ? (r >> 3) * 4 : 0;
    const bool half_ok = (r & 7) < M;
    const float* half_row = static_cast<const float*>(A) + static_cast<int64_t>(half_ok ? (r & 7) : 0) * lda;
    RawNormed ra0[kUnroll], ra1[kUnroll];
    bf16x8 w0[kUnroll][NT], w1[kUnroll][NT];
    auto issue = [&](RawNormed (&ra)[kUnroll], bf16x8 (&w)[kUnroll][NT], int first) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int k = (first + u * kWaves) * 32 + g * 8;
        const bool k_ok = k < K && first + u * kWaves < n_steps;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) w[u][nt] = load_frag(w_row[nt] + k, k_ok && w_ok[nt]);
        if constexpr (kHalf) {
          ra[u].lo = make_float4(0.f, 0.f, 0.f, 0.f);
          if (k_ok && half_ok) ra[u].lo = *reinterpret_cast<const float4*>(half_row + k + half_off);
        } else {
          load_raw(ra[u], a_row[0], k, k_ok && a_ok[0]);
        }
      }
    };
    auto multiply = [&](RawNormed (&ra)[kUnroll], bf16x8 (&w)[kUnroll][NT], int first) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int k = (first + u * kWaves) * 32 + g * 8;
        k = k < K ? k : 0;                   // (a step past the end holds zeros: any weights will do)
        bf16x8 a;
        if constexpr (kHalf) {
          const float4 x = ra[u].lo, nw = *reinterpret_cast<const float4*>(norm_lds + k + half_off);
          // (the squares of a row's eight values join its sum four and four, in lane r as in the plain form)
          const float sq = squares4(x), sq_other = lane_xor8(sq);
          if (r < 8) { ss[0] += sq; ss[0] += sq_other; }
          const uint32_t p0 = pack_bf16x2(x.x * nw.x, x.y * nw.y), p1 = pack_bf16x2(x.z * nw.z, x.w * nw.w);
          // the other four values of lane r's eight come from lane r + 8 (row_ror:8: every lane reads the lane eight on in its row of 16)
          const uint32_t q0 = __builtin_amdgcn_update_dpp(0u, p0, 0x128, 0xf, 0xf, false), q1 = __builtin_amdgcn_update_dpp(0u, p1, 0x128, 0xf, 0xf, false);
          const uint4 v = r < 8 ? make_uint4(p0, p1, q0, q1) : make_uint4(0, 0, 0, 0);      // (rows 8 to 15 of the tile do not exist)
          a = __builtin_bit_cast(bf16x8, v);
        } else {
          const RawNormed nw{*reinterpret_cast<const float4*>(norm_lds + k), *reinterpret_cast<const float4*>(norm_lds + k + 4)};
          a = to_frag(ra[u], nw, ss[0]);
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[0][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, w[u][nt], acc[0][nt], 0, 0, 0);
      }
    };
    constexpr int kStride = kUnroll * kWaves;
    int s = first_step + wave;
    issue(ra0, w0, s);
    issue(ra1, w1, s + kStride);
    for (int i = threadIdx.x * 4; i < K; i += kWaves * 64 * 4)
      *reinterpret_cast<float4*>(norm_lds + i) = *reinterpret_cast<const float4*>(norm_w + i);
    __syncthreads();
    for (; s < n_steps; s += 2 * kStride) {
      multiply(ra0, w0, s);
      issue(ra0, w0, s + 2 * kStride);
      multiply(ra1, w1, s + kStride);
      issue(ra1, w1, s + 3 * kStride);
    }
  }

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) red[wave][mt * NT + nt][lane] = acc[mt][nt];
  if constexpr (kNorm) {
    // the four lanes that hold slices of one row meet; the waves' shares of a row are added in wave order below
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const float row_ss = rows_sum(ss[mt]);      // (kHalf: lanes 8 to 15 of a row of lanes hold nothing, and stand for rows that do not exist)
      if (g == 0) ssq[wave][mt][r] = row_ss;
    }
  }
  __syncthreads();

  if (flat) {
    // one output a thread: the waves' shares in wave order, the same sums and the same arithmetic as below
    if (!f_ok) return;
    const float* shares = reinterpret_cast<const float*>(&red[0][0][0]);       // [wave][MT * NT][64 lanes][4]
    const int at = ((f_mt * NT + f_nt) * 64 + (f_g * 16 + f_r)) * 4 + f_i;
    float sum = shares[at], up = 0.f;
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sum += shares[w * (MT * NT * 256) + at];
    if (kEpilogue == kSkSwiglu) {
      up = shares[at + 256];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) up += shares[w * (MT * NT * 256) + at + 256];
    }
    if constexpr (kNorm) {
      float total = ssq[0][f_mt][f_g * 4 + f_i];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) total += ssq[w][f_mt][f_g * 4 + f_i];
      const float factor = __builtin_amdgcn_rsqf(total / static_cast<float>(K) + eps);
      sum *= factor;
      up *= factor;
    }
    TO* dst = out + static_cast<int64_t>(f_m) * ldo + f_n;
    if (kEpilogue == kSkStore) {
      store_f32(dst, sum + f_add);
    } else if (kEpilogue == kSkResidual) {
      store_f32(dst, f_add + sum);
    } else {
      store_f32(dst, sum / (1.f + __expf(-sum)) * up);
    }
    return;
  }

  if (k_splits > 1) {
    // this block's tiles (its waves added in wave order) go to the workspace; the last block to arrive goes on
    f32x4* mine = ws + (static_cast<int64_t>(blockIdx.x) * k_splits + blockIdx.y) * (MT * NT * 64);
    for (int tile = wave; tile < MT * NT; tile += kWaves) {
      f32x4 sum = red[0][tile][lane];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) sum += red[w][tile][lane];
      store_partial(mine + tile * 64 + lane, sum);
    }
    // Every wave waits until its partial sums have been performed in memory; only then may the
    // block be counted. A release fence of workgroup scope does not wait for stores to memory (the
    // counter could overtake them), and one of device scope writes this die's whole L2 back (measured with such
    // fences in every hand-over of this library: a decode step of 32 requests 2.81 instead of 1.24 ms). What makes the
    // hand-over sound here is the memory, not a fence: the workspace is uncached, the partial sums are stored and
    // read at device scope (past the L2s), and the counter is bumped only after every store has been acknowledged.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {
      const int arrived = atomicAdd(&counters[blockIdx.x], 1);
      last_block = arrived == k_splits - 1;
      if (last_block) atomicExch(&counters[blockIdx.x], 0);
    }
    __syncthreads();
    if (!last_block) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  }
  const f32x4* parts = ws + static_cast<int64_t>(blockIdx.x) * k_splits * (MT * NT * 64);

  // tiles are shared out among the waves; each adds the partial sums in wave (or split) order
#pragma unroll
  for (int it = 0; it < kMyTiles; ++it) {
    const int tile = wave + it * kWaves;
    if (tile >= kOutTiles) break;
    const int mt = (kEpilogue == kSkSwiglu) ? tile : tile / NT;
    const int nt = (kEpilogue == kSkSwiglu) ? 0 : tile % NT;
    f32x4 sum, up = f32x4{0.f, 0.f, 0.f, 0.f};
    if (k_splits > 1) {
      // (all the splits' loads on their way together, two, four or eight: they come from memory, and one after
      // the other each is waited for by itself; the order of the additions stays)
      const f32x4* first = parts + (mt * NT + nt) * 64 + lane;
      auto in_order = [&](auto count) {
        constexpr int kCount = decltype(count)::value;
        f32x4 theirs[kCount];
#pragma unroll
        for (int ks = 0; ks < kCount; ++ks) theirs[ks] = first[ks * MT * NT * 64];
        f32x4 total = theirs[0];
#pragma unroll
        for (int ks = 1; ks < kCount; ++ks) total += theirs[ks];
        return total;
      };
      if (k_splits == 2) sum = in_order(std::integral_constant<int, 2>());
      else if (k_splits == 4) sum = in_order(std::integral_constant<int, 4>());
      else sum = in_order(std::integral_constant<int, 8>());     // (the splits are doubled from one up to eight)
    } else {
      sum = red[0][mt * NT + nt][lane];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) sum += red[w][mt * NT + nt][lane];
      if (kEpilogue == kSkSwiglu) {
        up = red[0][mt * NT + 1][lane];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) up += red[w][mt * NT + 1][lane];
      }
    }
    const int n = (kEpilogue == kSkSwiglu) ? n0 + r : n0 + nt * 16 + r;
    if (n >= N || n - n0 >= cols) continue;
    if constexpr (kNorm) {
      // rows 4 g .. 4 g + 3 of the tile: their factors 1 / sqrt(mean of squares + eps)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float total = ssq[0][mt][g * 4 + i];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) total += ssq[w][mt][g * 4 + i];
        // (the hardware's reciprocal square root, good to one unit in the last place: an exact root and an exact
        // division are some hundred dependent instructions in a kernel that lasts a few microseconds)
        const float factor = __builtin_amdgcn_rsqf(total / static_cast<float>(K) + eps);
        sum[i] *= factor;
        up[i] *= factor;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = mt * 16 + g * 4 + i;
      if (m >= M) continue;
      TO* dst = out + static_cast<int64_t>(m) * ldo + n;
      if (kEpilogue == kSkStore) {
        store_f32(dst, sum[i] + add[it][i]);
      } else if (kEpilogue == kSkResidual) {
        store_f32(dst, add[it][i] + sum[i]);
      } else {
        const float gv = sum[i];
        store_f32(dst, gv / (1.f + __expf(-gv)) * up[i]);
      }
    }
  }
}

constexpr int kMaxNormK = 8192;    // columns of a product that takes a norm (the norm's weights lie in LDS)

struct NormArgs {
  const float* weight;   // null: A is bfloat16 and no norm is applied
  float eps;
};

// Parts of K that the blocks of a column tile share out (1: no hand-over through the workspace). A block reads its
// columns of W and every row of A over its share of K; a compute unit takes that in at a steady rate, the blocks come
// in rounds of one a compute unit (a round of four tiles of rows costs what 10 KB more would), and handing partial
// tiles over costs what 44 KB of reading do with two parts, 76 with four, 140 with eight. The parts are 1, 2, 4 or 8
// (every wave keeps a step): the number for which rounds x bytes a block + hand-over is least. The figures are fitted
// to 45 measured shapes (projections of the 0.5B to 32B sizes against 6 to 64 rows, each in 1, 2, 4 and 8 parts): the
// choice is the fastest or within 3 % of it for all but one matrix (2,048 x 11,008: two parts where four are 12 %
// faster). QKV of 1,152 x 896 stays whole up to 32 rows (5.3-5.6 us where two parts take 6.0-6.1) and goes in two parts
// from 48 on (64 rows 6.8 against 7.4); 2,048 x 2,048 against 32 rows goes in two parts (7.7 us; four, which outnumber
// the compute units, 11.0); 2,560 x 2,048 against 64 rows stays whole (13.5; eight parts 18.0).
template <int MT, int NT, int kWaves, int kEpilogue>
static int skinny_splits(int M, int N, int K) {
  constexpr int cols = (kEpilogue == kSkSwiglu) ? 16 : 16 * NT;
  const int col_tiles = (N + cols - 1) / cols;
  const Workspace& g_ws = workspace();
  if (kEpilogue == kSkSwiglu || g_ws.tiles == nullptr || col_tiles > kGemmCounters) return 1;
  const int steps = (K + 31) / 32, units = compute_units();
  const int64_t block_bytes = static_cast<int64_t>(M + cols) * K * 2;
  auto cost = [&](int parts) {
    const int64_t rounds = (static_cast<int64_t>(col_tiles) * parts + units - 1) / units;
    return rounds * (block_bytes / parts + (MT == 4 ? 10 : 0) * 1024) + (parts > 1 ? (12 + 16 * parts) * 1024 : 0);
  };
  int k_splits = 1;
  for (int parts = 2; parts <= 8 && steps / parts >= kWaves; parts *= 2) {
    if (static_cast<int64_t>(col_tiles) * parts * MT * NT * 256 > g_ws.tile_floats) break;
    if (cost(parts) < cost(k_splits)) k_splits = parts;
  }
  return k_splits;
}

template <int MT, int NT, int kWaves, int kEpilogue, typename TO>
static int launch_skinny(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                         const float* bias, int M, int N, int K, NormArgs norm, hipStream_t stream, int* splits_only) {
  constexpr int cols = (kEpilogue == kSkSwiglu) ? 16 : 16 * NT;
  const int col_tiles = (N + cols - 1) / cols;
  const Workspace& g_ws = workspace();
  if (splits_only) {
    *splits_only = skinny_splits<MT, NT, kWaves, kEpilogue>(M, N, K);
    return 0;
  }
  // (K is shared out over blocks only without a norm: the norm's sum of squares wants whole rows)
  const int k_splits = norm.weight == nullptr ? skinny_splits<MT, NT, kWaves, kEpilogue>(M, N, K) : 1;
  // loads in flight: many for one row tile (latency is all there is), fewer as row tiles take the registers
  constexpr int unroll = (MT >= 4) ? 2 : 4;
  if constexpr (kEpilogue != kSkResidual && sizeof(TO) == 2 && MT == 1) {
    if (norm.weight != nullptr) {
      // (float rows take twice the registers: two sets of two steps keep two blocks on a compute unit)
      ALOFA_REQUIRE(K % 4 == 0 && K <= kMaxNormK, "gemm_skinny: the norm's weights must fit in LDS [K=%d, at most %d]", K, kMaxNormK);
      // A compute unit takes in what its blocks read (the weights of their columns and, each block, all the rows) at
      // some 30 GB/s when all of them pull from memory, and the one with the most decides. So a block owns the number
      // of columns, a quarter of its tiles' to all of them, for which the most a compute unit reads is least (fewer
      // columns than all only for a tenth less): gate and up of 4,864 columns against eight rows of 896 in 487 blocks
      // of ten columns, two a compute unit, 7.4 us where 304 blocks of sixteen take 8.8 and 608 of eight 8.9; QKV of
      // 1,152 columns against sixteen rows in 231 blocks of five instead of 72 of sixteen (a decode step at batch 16
      // 0.930 against 0.938 ms).
      int own = cols;
      {
        const int64_t row_bytes = static_cast<int64_t>(M) * K * 4, col_bytes = static_cast<int64_t>(kEpilogue == kSkSwiglu ? 2 : 1) * K * 2;
        auto reads = [&](int c) {
          const int64_t blocks = (N + c - 1) / c, each = (blocks + compute_units() - 1) / compute_units();
          return each * (c * col_bytes + row_bytes);
        };
        for (int c = cols - 1; c >= cols / 4; --c)
          if (reads(c) * 10 < reads(own) * 9 || (reads(c) < reads(own) && own < cols)) own = c;
      }
      const int own_tiles = (N + own - 1) / own;
      if (M <= 8)
        gemm_skinny_kernel<MT, NT, kWaves, kEpilogue, TO, 2, 2><<<dim3(own_tiles, 1), kWaves * 64, K * sizeof(float), stream>>>(
            static_cast<TO*>(out), ldo, A, lda, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2), ldw, bias, M, N, K,
            reinterpret_cast<f32x4*>(g_ws.tiles), g_ws.counters, norm.weight, norm.eps, own);
      else
        gemm_skinny_kernel<MT, NT, kWaves, kEpilogue, TO, 2, 1><<<dim3(own_tiles, 1), kWaves * 64, K * sizeof(float), stream>>>(
            static_cast<TO*>(out), ldo, A, lda, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2), ldw, bias, M, N, K,
            reinterpret_cast<f32x4*>(g_ws.tiles), g_ws.counters, norm.weight, norm.eps, own);
      return check_launch("gemm_skinny (with norm)");
    }
  }
  ALOFA_REQUIRE(norm.weight == nullptr, "gemm_skinny: the norm goes with at most 16 rows and the bfloat16 store and swiglu epilogues only");
  gemm_skinny_kernel<MT, NT, kWaves, kEpilogue, TO, unroll, false><<<dim3(col_tiles, k_splits), kWaves * 64, 0, stream>>>(
      static_cast<TO*>(out), ldo, A, lda, static_cast<const bf16_t*>(W),
      static_cast<const bf16_t*>(W2), ldw, bias, M, N, K, reinterpret_cast<f32x4*>(g_ws.tiles), g_ws.counters, nullptr, 0.f, cols);
  return check_launch("gemm_skinny");
}

template <int kEpilogue, typename TO>
static int dispatch_skinny(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                           const float* bias, int M, int N, int K, NormArgs norm, hipStream_t stream, int* splits_only = nullptr) {
  // few columns: one 16-column tile per block and eight waves along K keep more of the chip busy;
  // many columns and many rows: four column tiles per block, so that the rows are read less often
  const bool narrow = (kEpilogue != kSkSwiglu) && N <= 4096;
#define ALOFA_SKINNY(MT, WIDE)                                                                                        \
  if (kEpilogue == kSkSwiglu)                                                                                         \
    return launch_skinny<MT, 2, (MT >= 4 ? 4 : 8), kEpilogue, TO>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm, stream, splits_only); \
  if (narrow) return launch_skinny<MT, 1, 8, kEpilogue, TO>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm, stream, splits_only);     \
  return launch_skinny<MT, WIDE, 4, kEpilogue, TO>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm, stream, splits_only);
  if (M <= 16) { ALOFA_SKINNY(1, 2) }
  if (M <= 32) { ALOFA_SKINNY(2, 4) }
  ALOFA_SKINNY(4, 4)
#undef ALOFA_SKINNY
}

}  // namespace alofa

using namespace alofa;

// Parts of K that alofa_gemm_skinny would share out over blocks for these sizes (1: none).
extern "C" int alofa_gemm_skinny_splits(int o_dtype, int M, int N, int K, int epilogue) {
  int splits = 1;
  const NormArgs none{nullptr, 0.f};
  if (M <= 0 || M > 64) return 1;
  if (epilogue == kSkStore && o_dtype == kBF16) dispatch_skinny<kSkStore, bf16_t>(nullptr, 0, nullptr, 0, nullptr, nullptr, 0, nullptr, M, N, K, none, nullptr, &splits);
  if (epilogue == kSkStore && o_dtype == kF32) dispatch_skinny<kSkStore, float>(nullptr, 0, nullptr, 0, nullptr, nullptr, 0, nullptr, M, N, K, none, nullptr, &splits);
  if (epilogue == kSkResidual) dispatch_skinny<kSkResidual, float>(nullptr, 0, nullptr, 0, nullptr, nullptr, 0, nullptr, M, N, K, none, nullptr, &splits);
  return splits;
}

// bfloat16 A [M, K] (M <= 64) and W [N, K] (W2 for the swiglu epilogue); K a multiple of 8,
// rows 16-byte aligned. Epilogues: 0 store (+ bias) as o_dtype, 1 add to the float residual, 2 swiglu.
// norm_w (float [K]) not null: A is float [M, K] and takes an RMSNorm with these weights and eps on
// its way into the product (bfloat16 store and swiglu epilogues; K is then not shared out over blocks).
extern "C" int alofa_gemm_skinny(void* out, int o_dtype, int64_t ldo, const void* A, int64_t lda, const void* W,
                                 const void* W2, int64_t ldw, const float* bias, int M, int N, int K, int epilogue,
                                 const float* norm_w, float eps, hipStream_t stream) {
  const NormArgs norm{norm_w, eps};
  ALOFA_REQUIRE(norm_w == nullptr || (reinterpret_cast<uintptr_t>(norm_w) % 16 == 0 && lda % 4 == 0 && eps > 0.f),
                "gemm_skinny: the norm's weights must be 16-byte aligned, eps positive");
  ALOFA_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: M=%d (1..64) N=%d K=%d", M, N, K);
  ALOFA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_skinny: K=%d, lda=%lld, ldw=%lld must be multiples of 8", K,
                static_cast<long long>(lda), static_cast<long long>(ldw));
  ALOFA_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(W2) % 16 == 0, "gemm_skinny: operands must be 16-byte aligned");
  ALOFA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_skinny: a leading dimension is shorter than its row");
  if (epilogue == kSkStore && o_dtype == kBF16)
    return dispatch_skinny<kSkStore, bf16_t>(out, ldo, A, lda, W, nullptr, ldw, bias, M, N, K, norm, stream);
  if (epilogue == kSkStore && o_dtype == kF32)
    return dispatch_skinny<kSkStore, float>(out, ldo, A, lda, W, nullptr, ldw, bias, M, N, K, norm, stream);
  if (epilogue == kSkResidual && o_dtype == kF32)
    return dispatch_skinny<kSkResidual, float>(out, ldo, A, lda, W, nullptr, ldw, nullptr, M, N, K, norm, stream);
  if (epilogue == kSkSwiglu && o_dtype == kBF16) {
    ALOFA_REQUIRE(W2 != nullptr, "gemm_skinny: the swiglu epilogue needs the up matrix");
    return dispatch_skinny<kSkSwiglu, bf16_t>(out, ldo, A, lda, W, W2, ldw, nullptr, M, N, K, norm, stream);
  }
  ALOFA_REQUIRE(false, "gemm_skinny: unsupported epilogue %d with out dtype %d", epilogue, o_dtype);
}
