// Matrix products for at most eight rows (the decode steps of few requests), bfloat16, on the
// vector units: out[m, n] = sum_k A[m, k] * W[n, k] with M <= 8 (M <= 16 for plain products: bfloat16 rows,
// store or residual epilogue, K <= 6144).
//
// The work is streaming W once from memory, and the time is what a compute unit needs to pull
// its share, so the shares are made small and even: a block owns C output columns (rows of W,
// four or eight), however few columns there are, and its wavefronts cut K into runs of 512:
// lane l of wave w holds the eight values 512 w + 8 l .. + 7 of every row of A and of each of
// the block's rows of W (one 16-byte load each, a wave's loads of a row contiguous), multiplies
// them in pairs (v_dot2_f32_bf16, float sums) and keeps C * M partial sums. Nothing is waited
// for before every load of the block is on its way, and no block waits for another: where the
// matrix-core kernel for few rows needs sixteen columns per block and, for a matrix of few
// columns, a hand-over of partial sums between blocks through memory, this one needs neither.
//
// The lanes' partial sums meet by exchange: at distance 32, 16, 8, 4, 2 the lanes swap one half
// of their values and add, so that each keeps half as many, then the last pair is added; the
// waves' sums meet in LDS and are added in wave order. The order of additions is fixed and the
// same for every row whatever else is in the batch (M only selects how many rows are computed).
//
// Up to twelve runs of 512 a wave takes one run (no loop at all); a longer K (the down projection of
// a wide feed-forward) goes to a second kernel whose eight waves take every eighth run in turn, the loads
// of the next run on their way while this one is multiplied.
//
// With a norm (kNorm) the rows of A are the float residual stream: a value is x * w_norm rounded
// to bfloat16, the squares of x are summed beside the products, and the row's factor
// 1 / sqrt(mean + eps) multiplies the finished sum, as in the matrix-core kernel for few rows.
#include "common.h"

namespace alofa {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

enum RowsEpilogue : int { kRwStore = 0, kRwResidual = 1, kRwSwiglu = 2 };

constexpr int kRowsMaxWaves = 12;     // runs of 512 along K, one per wave
constexpr int kRowsMaxK = kRowsMaxWaves * 512;

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

// v of lane l ^ 4 (within a row of 16): the lanes of banks 0 and 2 (four lanes each) read four lanes up,
// those of banks 1 and 3 four lanes down
__device__ __forceinline__ float lane_xor4(float v) {
  const uint32_t x = __float_as_uint(v);
  const uint32_t up = __builtin_amdgcn_update_dpp(0u, x, 0x104, 0xf, 0x5, false);     // row_shl:4 into banks 0, 2
  return __uint_as_float(__builtin_amdgcn_update_dpp(up, x, 0x114, 0xf, 0xa, false));   // row_shr:4 into banks 1, 3
}

// The sums over all 64 lanes of n values per lane (n a power of two, at most 64), by halving: after the
// step at distance d a lane whose bit d is set holds the upper half of the values, summed with its
// partner's, the other lane the lower half; the steps go from distance 32 down, and where one value is
// left it is added across the remaining distances. Afterwards v[0] of lane l is the total of value
// l >> (6 - log2 n). Every value goes through the same tree of lanes whatever n is.
template <int n, int d>
__device__ __forceinline__ void lanes_sum_step(float* v, int lane) {
  if constexpr (d >= 1) {
    if constexpr (n > 1) {
      constexpr int h = n / 2;
      const bool upper = (lane & d) != 0;
#pragma unroll
      for (int i = 0; i < h; ++i) {
        if constexpr (d == 32) {
          const auto s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[i]), __float_as_uint(v[i + h]), false, false);
          v[i] = __uint_as_float(s[0]) + __uint_as_float(s[1]);
        } else if constexpr (d == 16) {
          const auto s = __builtin_amdgcn_permlane16_swap(__float_as_uint(v[i]), __float_as_uint(v[i + h]), false, false);
          v[i] = __uint_as_float(s[0]) + __uint_as_float(s[1]);
        } else {
          const float send = upper ? v[i] : v[i + h];
          const float keep = upper ? v[i + h] : v[i];
          const float got = d == 8 ? lane_xor8(send) : d == 4 ? lane_xor4(send) : d == 2 ? lane_xor2(send) : lane_xor1(send);
          v[i] = keep + got;
        }
      }
      lanes_sum_step<h, d / 2>(v, lane);
    } else {
      if constexpr (d == 32) {
        const auto s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[0]), __float_as_uint(v[0]), false, false);
        v[0] = __uint_as_float(s[0]) + __uint_as_float(s[1]);
      } else if constexpr (d == 16) {
        const auto s = __builtin_amdgcn_permlane16_swap(__float_as_uint(v[0]), __float_as_uint(v[0]), false, false);
        v[0] = __uint_as_float(s[0]) + __uint_as_float(s[1]);
      } else {
        v[0] += d == 8 ? lane_xor8(v[0]) : d == 4 ? lane_xor4(v[0]) : d == 2 ? lane_xor2(v[0]) : lane_xor1(v[0]);
      }
      lanes_sum_step<1, d / 2>(v, lane);
    }
  }
}
template <int n>
__device__ __forceinline__ void lanes_sum(float (&v)[n], int lane) {
  static_assert(n >= 1 && n <= 64 && (n & (n - 1)) == 0, "a power of two of values, at most one per lane");
  lanes_sum_step<n, 32>(v, lane);
}
constexpr int log2_of(int n) { return n <= 1 ? 0 : 1 + log2_of(n / 2); }

// MR: rows computed (1, 2, 4, 8, or 16 for plain products; rows beyond M are not stored); C: columns per block; kRwSwiglu: W is the gate
// matrix and W2 the up matrix, same columns; TO: float or bf16_t; kMaxWaves: bound of the block's waves.
template <int MR, int C, int kEpilogue, typename TO, bool kNorm, int kMaxWaves>
__global__ void __launch_bounds__(64 * kMaxWaves) gemm_rows_kernel(
    TO* __restrict__ out, int64_t ldo, const void* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W,
    const bf16_t* __restrict__ W2, int64_t ldw, const float* __restrict__ bias, int M, int N, int K,
    const float* __restrict__ norm_w, float eps) {
  constexpr int kMats = (kEpilogue == kRwSwiglu) ? 2 : 1;
  constexpr int V = C * MR;                                // partial sums per lane and matrix
  __shared__ float red[kMaxWaves][kMats][V];
  __shared__ float ssq[kNorm ? kMaxWaves : 1][MR];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, n_waves = blockDim.x / 64;
  const int n0 = blockIdx.x * C;
  const int k0 = (wave * 64 + lane) * 8;
  const bool k_ok = k0 < K;

  // Every load of this lane sets out, the weights (from memory) first, then the rows (which every block reads:
  // from L2). No load is conditional: a lane past the end of K reads where lane 0 does, rows beyond M and columns
  // beyond N read the last row and column (what they give is cleared below, or never stored), so that the loads are
  // one straight run of instructions with nothing to wait for between them.
  const int k_at = k_ok ? k0 : 0;
  uint4 wv[kMats][C];
#pragma unroll
  for (int mat = 0; mat < kMats; ++mat)
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const bf16_t* base = mat == 0 ? W : W2;
      const int n = n0 + c < N ? n0 + c : N - 1;
      wv[mat][c] = *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(n) * ldw + k_at);
    }
  uint4 av[MR];               // the rows' values as pairs of bfloat16
  float4 xlo[kNorm ? MR : 1], xhi[kNorm ? MR : 1], nlo, nhi;
  if constexpr (kNorm) {
    nlo = *reinterpret_cast<const float4*>(norm_w + k_at);
    nhi = *reinterpret_cast<const float4*>(norm_w + k_at + 4);
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float* row = static_cast<const float*>(A) + static_cast<int64_t>(m < M ? m : M - 1) * lda + k_at;
      xlo[m] = *reinterpret_cast<const float4*>(row);
      xhi[m] = *reinterpret_cast<const float4*>(row + 4);
    }
  } else {
#pragma unroll
    for (int m = 0; m < MR; ++m)
      av[m] = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(A) + static_cast<int64_t>(m < M ? m : M - 1) * lda + k_at);
  }
  // what the epilogue adds sets out too: thread c * MR + m finishes out[m, n0 + c]
  const int my_c = threadIdx.x / MR, my_m = threadIdx.x % MR;
  const bool finisher = threadIdx.x < V && my_m < M && n0 + my_c < N;
  float add = 0.f;
  if (finisher) {
    if (kEpilogue == kRwStore && bias) add = bias[n0 + my_c];
    if (kEpilogue == kRwResidual) add = load_f32(out + static_cast<int64_t>(my_m) * ldo + n0 + my_c);
  }
  // a lane past the end of K adds nothing: its weights and its rows' values are cleared
  if (!k_ok) {
#pragma unroll
    for (int mat = 0; mat < kMats; ++mat)
#pragma unroll
      for (int c = 0; c < C; ++c) wv[mat][c] = make_uint4(0, 0, 0, 0);
    if constexpr (kNorm) {
#pragma unroll
      for (int m = 0; m < MR; ++m) xlo[m] = xhi[m] = make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
#pragma unroll
      for (int m = 0; m < MR; ++m) av[m] = make_uint4(0, 0, 0, 0);
    }
  }

  float ss[MR];
  if constexpr (kNorm) {
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float4 a = xlo[m], b = xhi[m];
      ss[m] = a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
      ss[m] += b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
      av[m] = make_uint4(pack_bf16x2(a.x * nlo.x, a.y * nlo.y), pack_bf16x2(a.z * nlo.z, a.w * nlo.w),
                         pack_bf16x2(b.x * nhi.x, b.y * nhi.y), pack_bf16x2(b.z * nhi.z, b.w * nhi.w));
    }
  }

  float acc[kMats][V];
#pragma unroll
  for (int mat = 0; mat < kMats; ++mat)
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        float s = dot2(av[m].x, wv[mat][c].x, 0.f);
        s = dot2(av[m].y, wv[mat][c].y, s);
        s = dot2(av[m].z, wv[mat][c].z, s);
        acc[mat][c * MR + m] = dot2(av[m].w, wv[mat][c].w, s);
      }

  // the lanes' sums meet; lane l then holds value l >> kShift
  constexpr int kShift = 6 - log2_of(V);
#pragma unroll
  for (int mat = 0; mat < kMats; ++mat) {
    lanes_sum<V>(acc[mat], lane);
    if ((lane & ((1 << kShift) - 1)) == 0) red[wave][mat][lane >> kShift] = acc[mat][0];
  }
  if constexpr (kNorm) {
    lanes_sum<MR>(ss, lane);
    constexpr int kRowShift = 6 - log2_of(MR);
    if ((lane & ((1 << kRowShift) - 1)) == 0) ssq[wave][lane >> kRowShift] = ss[0];
  }
  __syncthreads();

  if (!finisher) return;
  float sum = red[0][0][threadIdx.x], up = 0.f;
  for (int w = 1; w < n_waves; ++w) sum += red[w][0][threadIdx.x];
  if constexpr (kEpilogue == kRwSwiglu) {
    up = red[0][1][threadIdx.x];
    for (int w = 1; w < n_waves; ++w) up += red[w][1][threadIdx.x];
  }
  if constexpr (kNorm) {
    float total = ssq[0][my_m];
    for (int w = 1; w < n_waves; ++w) total += ssq[w][my_m];
    // (the hardware's reciprocal square root, good to one unit in the last place, as in the matrix-core kernel)
    const float factor = __builtin_amdgcn_rsqf(total / static_cast<float>(K) + eps);
    sum *= factor;
    up *= factor;
  }
  TO* dst = out + static_cast<int64_t>(my_m) * ldo + n0 + my_c;
  if (kEpilogue == kRwStore) {
    store_f32(dst, sum + add);
  } else if (kEpilogue == kRwResidual) {
    store_f32(dst, add + sum);
  } else {
    store_f32(dst, sum / (1.f + __expf(-sum)) * up);
  }
}

// K beyond kRowsMaxK: the block's eight waves (eight rows' operands leave no registers for more, and the number
// must not depend on the rows: it sets the order of the additions) take the runs wave, wave + 8, ... in turn, two
// sets of operands
// in flight (each is loaded again as soon as it has been multiplied: no copies between sets, a copy would wait
// for its load). Store and residual epilogues, bfloat16 rows.
constexpr int rows_long_waves(int) { return 8; }

template <int MR, int C, int kEpilogue, typename TO>
__global__ void __launch_bounds__(64 * rows_long_waves(MR)) gemm_rows_long_kernel(
    TO* __restrict__ out, int64_t ldo, const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W, int64_t ldw,
    const float* __restrict__ bias, int M, int N, int K) {
  constexpr int V = C * MR, kWaves = rows_long_waves(MR);
  __shared__ float red[kWaves][V];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int n0 = blockIdx.x * C;
  const bf16_t* w_row[C];
  const bf16_t* a_row[MR];
#pragma unroll
  for (int c = 0; c < C; ++c) w_row[c] = W + static_cast<int64_t>(n0 + c < N ? n0 + c : N - 1) * ldw;
#pragma unroll
  for (int m = 0; m < MR; ++m) a_row[m] = A + static_cast<int64_t>(m < M ? m : M - 1) * lda;
  struct Set {
    uint4 w[C], a[MR];
  };
  // run `run` of K sets out (a lane past the end of K reads where lane 0 of the first run does; cleared at use)
  auto fetch = [&](Set& s, int run) __attribute__((always_inline)) {
    const int k0 = (run * 64 + lane) * 8;
    const int k_at = k0 < K ? k0 : 0;
#pragma unroll
    for (int c = 0; c < C; ++c) s.w[c] = *reinterpret_cast<const uint4*>(w_row[c] + k_at);
#pragma unroll
    for (int m = 0; m < MR; ++m) s.a[m] = *reinterpret_cast<const uint4*>(a_row[m] + k_at);
  };
  float acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = 0.f;
  auto multiply = [&](const Set& s, int run) __attribute__((always_inline)) {
    const bool k_ok = (run * 64 + lane) * 8 < K;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const uint4 w = k_ok ? s.w[c] : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        float t = dot2(s.a[m].x, w.x, acc[c * MR + m]);
        t = dot2(s.a[m].y, w.y, t);
        t = dot2(s.a[m].z, w.z, t);
        acc[c * MR + m] = dot2(s.a[m].w, w.w, t);
      }
    }
  };
  const int my_c = threadIdx.x / MR, my_m = threadIdx.x % MR;
  const bool finisher = threadIdx.x < V && my_m < M && n0 + my_c < N;
  float add = 0.f;
  if (finisher) {
    if (kEpilogue == kRwStore && bias) add = bias[n0 + my_c];
    if (kEpilogue == kRwResidual) add = load_f32(out + static_cast<int64_t>(my_m) * ldo + n0 + my_c);
  }
  const int runs = (K + 511) / 512;
  Set s0, s1;
  int run = wave;
  fetch(s0, run);
  fetch(s1, run + kWaves);
  // (whole rounds: every fetch is issued, a run past the end reads run 0's place and adds nothing)
  for (; run < runs; run += 2 * kWaves) {
    multiply(s0, run);
    fetch(s0, run + 2 * kWaves);
    multiply(s1, run + kWaves);
    fetch(s1, run + 3 * kWaves);
  }
  constexpr int kShift = 6 - log2_of(V);
  lanes_sum<V>(acc, lane);
  if ((lane & ((1 << kShift) - 1)) == 0) red[wave][lane >> kShift] = acc[0];
  __syncthreads();
  if (!finisher) return;
  float sum = red[0][threadIdx.x];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) sum += red[w][threadIdx.x];
  TO* dst = out + static_cast<int64_t>(my_m) * ldo + n0 + my_c;
  store_f32(dst, kEpilogue == kRwStore ? sum + add : add + sum);
}

template <int MR, int C, int kEpilogue, typename TO, bool kNorm>
static int launch_rows(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                       const float* bias, int M, int N, int K, const float* norm_w, float eps, hipStream_t stream) {
  const int waves = (K + 511) / 512;
  const dim3 grid((N + C - 1) / C);
  if (waves > kRowsMaxWaves) {
    if constexpr (!kNorm && kEpilogue != kRwSwiglu && MR <= 8) {
      gemm_rows_long_kernel<MR, C, kEpilogue, TO><<<grid, 64 * rows_long_waves(MR), 0, stream>>>(
          static_cast<TO*>(out), ldo, static_cast<const bf16_t*>(A), lda, static_cast<const bf16_t*>(W), ldw, bias, M, N, K);
      return check_launch("gemm_rows (long K)");
    }
    ALOFA_REQUIRE(false, "gemm_rows: K=%d beyond %d goes with the store and residual epilogues of bfloat16 rows only", K, kRowsMaxK);
    return 1;
  }
#define ALOFA_ROWS(MAXW)                                                                                               \
  gemm_rows_kernel<MR, C, kEpilogue, TO, kNorm, MAXW><<<grid, 64 * waves, 0, stream>>>(                                \
      static_cast<TO*>(out), ldo, A, lda, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2), ldw, bias, M, \
      N, K, norm_w, eps)
  if (waves <= 4) {
    ALOFA_ROWS(4);
  } else {
    ALOFA_ROWS(kRowsMaxWaves);
  }
#undef ALOFA_ROWS
  return check_launch("gemm_rows");
}

template <int kEpilogue, typename TO, bool kNorm>
static int dispatch_rows(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                         const float* bias, int M, int N, int K, const float* norm_w, float eps, hipStream_t stream) {
  // (gate and up: eight columns of either, so that the rows, which every block reads and, with a norm, converts,
  // are read half as often where the blocks are many)
  constexpr int C = (kEpilogue == kRwSwiglu) ? 8 : 4;
  if (M <= 1) return launch_rows<1, C, kEpilogue, TO, kNorm>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm_w, eps, stream);
  if (M <= 2) return launch_rows<2, C, kEpilogue, TO, kNorm>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm_w, eps, stream);
  if (M <= 4) return launch_rows<4, C, kEpilogue, TO, kNorm>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm_w, eps, stream);
  if constexpr (!kNorm && kEpilogue != kRwSwiglu) {
    if (M > 8) return launch_rows<16, C, kEpilogue, TO, kNorm>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm_w, eps, stream);
  }
  return launch_rows<8, C, kEpilogue, TO, kNorm>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm_w, eps, stream);
}

}  // namespace alofa

using namespace alofa;

// Whether alofa_gemm_rows takes these sizes.
// (K beyond 6,144, or nine to sixteen rows: the store and residual epilogues of bfloat16 rows only, `plain` then says
// that this is such a product)
extern "C" int alofa_gemm_rows_fits(int M, int N, int K, int plain) {
  return M >= 1 && (M <= 8 || (plain && M <= 16 && K <= kRowsMaxK)) && N >= 1 && K >= 8 && K % 8 == 0 && (K <= kRowsMaxK || plain);
}

// The same operands and epilogues as alofa_gemm_skinny (bfloat16 A [M, K] and W [N, K]; W2 for the swiglu epilogue;
// 0 store (+ bias) as o_dtype, 1 add to the float residual, 2 swiglu; norm_w not null: A is float [M, K] and takes
// an RMSNorm with these weights and eps on its way, bfloat16 store and swiglu epilogues), for M <= 8; K beyond 6,144
// with the store and residual epilogues of bfloat16 rows only.
extern "C" int alofa_gemm_rows(void* out, int o_dtype, int64_t ldo, const void* A, int64_t lda, const void* W,
                               const void* W2, int64_t ldw, const float* bias, int M, int N, int K, int epilogue,
                               const float* norm_w, float eps, hipStream_t stream) {
  ALOFA_REQUIRE(alofa_gemm_rows_fits(M, N, K, norm_w == nullptr && epilogue != kRwSwiglu),
                "gemm_rows: M=%d (1..8; to 16 for plain products of K up to 6,144) N=%d K=%d (a multiple of 8; beyond %d with the store and residual epilogues of bfloat16 rows only)", M, N, K, kRowsMaxK);
  ALOFA_REQUIRE(ldw % 8 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 && (W2 == nullptr || reinterpret_cast<uintptr_t>(W2) % 16 == 0),
                "gemm_rows: rows of W must be 16-byte aligned");
  ALOFA_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && lda % (norm_w ? 4 : 8) == 0, "gemm_rows: rows of A must be 16-byte aligned");
  ALOFA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_rows: strides shorter than the rows");
  ALOFA_REQUIRE(norm_w == nullptr || (reinterpret_cast<uintptr_t>(norm_w) % 16 == 0 && eps > 0.f), "gemm_rows: the norm's weights must be 16-byte aligned, eps positive");
  if (norm_w != nullptr) {
    if (epilogue == kRwStore && o_dtype == kBF16) return dispatch_rows<kRwStore, bf16_t, true>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm_w, eps, stream);
    if (epilogue == kRwSwiglu && o_dtype == kBF16 && W2) return dispatch_rows<kRwSwiglu, bf16_t, true>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, norm_w, eps, stream);
    ALOFA_REQUIRE(false, "gemm_rows: the norm goes with the bfloat16 store and swiglu epilogues only");
    return 1;
  }
  if (epilogue == kRwStore && o_dtype == kBF16) return dispatch_rows<kRwStore, bf16_t, false>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, nullptr, 0.f, stream);
  if (epilogue == kRwStore && o_dtype == kF32) return dispatch_rows<kRwStore, float, false>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, nullptr, 0.f, stream);
  if (epilogue == kRwResidual && o_dtype == kF32) return dispatch_rows<kRwResidual, float, false>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, nullptr, 0.f, stream);
  if (epilogue == kRwSwiglu && o_dtype == kBF16 && W2) return dispatch_rows<kRwSwiglu, bf16_t, false>(out, ldo, A, lda, W, W2, ldw, bias, M, N, K, nullptr, 0.f, stream);
  ALOFA_REQUIRE(false, "gemm_rows: no kernel for epilogue %d with output type %d", epilogue, o_dtype);
  return 1;
}
