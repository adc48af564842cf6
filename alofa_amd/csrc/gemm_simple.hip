// General matrix products out[m, n] = sum_k A[m, k] * W[n, k] for any sizes and
// any mix of float / bfloat16 operands. W is stored [out, in] (row n holds the
// weights of output n), so nothing is transposed at load.
//
// Every output element has one accumulator that starts at the bias and takes
// the products in ascending k, whatever M is and wherever the row lies in the
// batch: a row's result does not depend on what else is computed with it.
// Acc = double gives the float32 model with float64 accumulation; Acc = float is
// the plain float path. These kernels are the slow, always-valid path; the
// MFMA and skinny kernels take over where their shapes fit.
#include "common.h"

namespace alofa {

enum Epilogue : int { kStore = 0, kAddToResidual = 1 };

constexpr int BM = 64, BN = 64, BK = 16;

template <typename TA, typename TW, typename Acc>
__device__ __forceinline__ void load_tiles(Acc (*As)[BM + 1], Acc (*Ws)[BN + 1], const TA* A, int64_t lda,
                                           const TW* W, int64_t ldw, int m0, int n0, int k0, int M, int N, int K) {
  // 256 threads move 64x16 of A and 64x16 of W; consecutive threads read consecutive k
  for (int i = threadIdx.x; i < BM * BK; i += 256) {
    const int r = i / BK, c = i % BK;
    const int m = m0 + r, k = k0 + c;
    As[c][r] = (m < M && k < K) ? static_cast<Acc>(load_f32(A + static_cast<int64_t>(m) * lda + k)) : Acc(0);
  }
  for (int i = threadIdx.x; i < BN * BK; i += 256) {
    const int r = i / BK, c = i % BK;
    const int n = n0 + r, k = k0 + c;
    Ws[c][r] = (n < N && k < K) ? static_cast<Acc>(load_f32(W + static_cast<int64_t>(n) * ldw + k)) : Acc(0);
  }
}

template <typename TA, typename TW, typename TO, typename Acc, int kEpilogue>
__global__ void __launch_bounds__(256) gemm_simple_kernel(TO* __restrict__ out, int64_t ldo, const TA* __restrict__ A,
                                                          int64_t lda, const TW* __restrict__ W, int64_t ldw,
                                                          const float* __restrict__ bias, int M, int N, int K) {
  __shared__ Acc As[BK][BM + 1];
  __shared__ Acc Ws[BK][BN + 1];
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  Acc acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      acc[i][j] = (bias && n < N) ? static_cast<Acc>(bias[n]) : Acc(0);
    }
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
    load_tiles<TA, TW, Acc>(As, Ws, A, lda, W, ldw, m0, n0, k0, M, N, K);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      Acc a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty + 16 * i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx + 16 * j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * w[j];
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty + 16 * i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      TO* dst = out + static_cast<int64_t>(m) * ldo + n;
      const float v = static_cast<float>(acc[i][j]);
      if (kEpilogue == kAddToResidual)
        store_f32(dst, load_f32(dst) + v);
      else
        store_f32(dst, v);
    }
  }
}

// out[m, n] = silu(A Wg^T)[m, n] * (A Wu^T)[m, n]: both products are rounded to
// float first, then x / (1 + exp(-x)) * u in Acc.
template <typename TA, typename TW, typename TO, typename Acc>
__global__ void __launch_bounds__(256) gemm_swiglu_simple_kernel(TO* __restrict__ out, int64_t ldo,
                                                                 const TA* __restrict__ A, int64_t lda,
                                                                 const TW* __restrict__ Wg, const TW* __restrict__ Wu,
                                                                 int64_t ldw, int M, int N, int K) {
  __shared__ Acc As[BK][BM + 1];
  __shared__ Acc Gs[BK][BN + 1];
  __shared__ Acc Us[BK][BN + 1];
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  Acc g[4][4], u[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) g[i][j] = u[i][j] = Acc(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
    load_tiles<TA, TW, Acc>(As, Gs, A, lda, Wg, ldw, m0, n0, k0, M, N, K);
    for (int i = threadIdx.x; i < BN * BK; i += 256) {
      const int r = i / BK, c = i % BK;
      const int n = n0 + r, k = k0 + c;
      Us[c][r] = (n < N && k < K) ? static_cast<Acc>(load_f32(Wu + static_cast<int64_t>(n) * ldw + k)) : Acc(0);
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      Acc a[4], wg[4], wu[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty + 16 * i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wg[j] = Gs[kk][tx + 16 * j];
        wu[j] = Us[kk][tx + 16 * j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          g[i][j] += a[i] * wg[j];
          u[i][j] += a[i] * wu[j];
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty + 16 * i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      const Acc gv = static_cast<Acc>(static_cast<float>(g[i][j]));
      const Acc uv = static_cast<Acc>(static_cast<float>(u[i][j]));
      store_f32(out + static_cast<int64_t>(m) * ldo + n, static_cast<float>(gv / (Acc(1) + exp(-gv)) * uv));
    }
  }
}

template <typename TA, typename TW, typename TO, typename Acc>
static int launch_gemm(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, int64_t ldw,
                       const float* bias, int M, int N, int K, int epilogue, hipStream_t stream) {
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (epilogue == kStore)
    gemm_simple_kernel<TA, TW, TO, Acc, kStore><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), ldo, static_cast<const TA*>(A), lda,
                                                                          static_cast<const TW*>(W), ldw, bias, M, N, K);
  else
    gemm_simple_kernel<TA, TW, TO, Acc, kAddToResidual><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), ldo, static_cast<const TA*>(A), lda,
                                                                                  static_cast<const TW*>(W), ldw, bias, M, N, K);
  return check_launch("gemm_simple");
}

template <typename TA, typename TW, typename TO, typename Acc>
static int launch_gemm_swiglu(void* out, int64_t ldo, const void* A, int64_t lda, const void* Wg, const void* Wu,
                              int64_t ldw, int M, int N, int K, hipStream_t stream) {
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  gemm_swiglu_simple_kernel<TA, TW, TO, Acc><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), ldo, static_cast<const TA*>(A), lda,
                                                                       static_cast<const TW*>(Wg), static_cast<const TW*>(Wu), ldw, M, N, K);
  return check_launch("gemm_swiglu_simple");
}

}  // namespace alofa

using namespace alofa;

// Dtypes: a = activations in, w = weights, o = out. exact != 0 needs all float.
extern "C" int alofa_gemm_simple(void* out, int o_dtype, int64_t ldo, const void* A, int a_dtype, int64_t lda,
                                 const void* W, int w_dtype, int64_t ldw, const float* bias, int M, int N, int K,
                                 int epilogue, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: M=%d N=%d K=%d must be positive", M, N, K);
  ALOFA_REQUIRE(epilogue == kStore || epilogue == kAddToResidual, "gemm: unknown epilogue %d", epilogue);
  ALOFA_REQUIRE(epilogue != kAddToResidual || o_dtype == kF32, "gemm: the residual stream is float");
  ALOFA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm: a leading dimension is shorter than its row");
  if (exact) {
    ALOFA_REQUIRE(a_dtype == kF32 && w_dtype == kF32 && o_dtype == kF32, "gemm: the exact path takes float operands only");
    return launch_gemm<float, float, float, double>(out, ldo, A, lda, W, ldw, bias, M, N, K, epilogue, stream);
  }
#define ALOFA_GEMM_CASE(ad, wd, od, TA, TW, TO) \
  if (a_dtype == ad && w_dtype == wd && o_dtype == od) \
    return launch_gemm<TA, TW, TO, float>(out, ldo, A, lda, W, ldw, bias, M, N, K, epilogue, stream);
  ALOFA_GEMM_CASE(kBF16, kBF16, kBF16, bf16_t, bf16_t, bf16_t)
  ALOFA_GEMM_CASE(kBF16, kBF16, kF32, bf16_t, bf16_t, float)
  ALOFA_GEMM_CASE(kBF16, kF32, kBF16, bf16_t, float, bf16_t)
  ALOFA_GEMM_CASE(kBF16, kF32, kF32, bf16_t, float, float)
  ALOFA_GEMM_CASE(kF32, kF32, kF32, float, float, float)
#undef ALOFA_GEMM_CASE
  ALOFA_REQUIRE(false, "gemm: unsupported dtype mix a=%d w=%d o=%d", a_dtype, w_dtype, o_dtype);
}

extern "C" int alofa_gemm_swiglu_simple(void* out, int o_dtype, int64_t ldo, const void* A, int a_dtype, int64_t lda,
                                        const void* Wg, const void* Wu, int w_dtype, int64_t ldw, int M, int N,
                                        int K, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_swiglu: M=%d N=%d K=%d must be positive", M, N, K);
  ALOFA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_swiglu: a leading dimension is shorter than its row");
  if (exact) {
    ALOFA_REQUIRE(a_dtype == kF32 && w_dtype == kF32 && o_dtype == kF32, "gemm_swiglu: the exact path takes float operands only");
    return launch_gemm_swiglu<float, float, float, double>(out, ldo, A, lda, Wg, Wu, ldw, M, N, K, stream);
  }
  if (a_dtype == kBF16 && w_dtype == kBF16 && o_dtype == kBF16)
    return launch_gemm_swiglu<bf16_t, bf16_t, bf16_t, float>(out, ldo, A, lda, Wg, Wu, ldw, M, N, K, stream);
  if (a_dtype == kBF16 && w_dtype == kF32 && o_dtype == kBF16)
    return launch_gemm_swiglu<bf16_t, float, bf16_t, float>(out, ldo, A, lda, Wg, Wu, ldw, M, N, K, stream);
  if (a_dtype == kF32 && w_dtype == kF32 && o_dtype == kF32)
    return launch_gemm_swiglu<float, float, float, float>(out, ldo, A, lda, Wg, Wu, ldw, M, N, K, stream);
  ALOFA_REQUIRE(false, "gemm_swiglu: unsupported dtype mix a=%d w=%d o=%d", a_dtype, w_dtype, o_dtype);
}
