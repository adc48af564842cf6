// Matrix products for many rows (prompt portions), bfloat16 on MFMA:
// out[m, n] = sum_k A[m, k] * W[n, k].
//
// A block of four wavefronts (2 x 2) computes a 128 x 128 tile of the output,
// every wave a 64 x 64 quarter as 2 x 2 tiles of v_mfma_f32_32x32x16_bf16; for
// outputs too small to fill the chip with such tiles the block computes 64 x 64
// (one MFMA tile per wave). Per step of 64 along K the block stages a slab of A
// and of W in LDS
// (16-byte loads along K; rows are padded by 8 elements so that the fragment
// reads fall on distinct banks), while the next slab is already on its way from
// memory into registers. Accumulation is float; each output element has one
// accumulator that takes the products in ascending k, whatever M is.
//
// Operand layout of the instruction, lane l: A holds row l % 32 and B column
// l % 32, both the reduction indices 8 * (l / 32) .. + 7 of the 16; D holds
// column l % 32 and, in acc[i], row 8 * (i / 4) + 4 * (l / 32) + i % 4.
//
// Epilogues: store (+ bias), add to the float residual stream, and SwiGLU, for
// which a block computes the gate and the up product of the same 64 columns
// (its W slab holds 64 rows of each) and writes silu(gate) * up.
#include "common.h"

namespace alofa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum MfmaEpilogue : int { kMfStore = 0, kMfResidual = 1, kMfSwiglu = 2 };

constexpr int TK = 64, PAD = 8;
constexpr int kRow = TK + PAD;  // LDS row length in elements

// WT: MFMA tiles per wave along each of m and n (2: 128 x 128 block tile, 1: 64 x 64).
// PF: slabs on their way from memory while another is being multiplied.
template <int kEpilogue, typename TO, int WT, int PF>
__global__ void __launch_bounds__(256) gemm_mfma_kernel(TO* __restrict__ out, int64_t ldo,
                                                        const bf16_t* __restrict__ A, int64_t lda,
                                                        const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
                                                        int64_t ldw, const float* __restrict__ bias, int M, int N,
                                                        int K) {
  constexpr int TM = 64 * WT, TN = 64 * WT;
  static_assert(kEpilogue != kMfSwiglu || WT == 2, "the swiglu epilogue needs two column tiles per wave");
  __shared__ __attribute__((aligned(16))) bf16_t As[TM * kRow];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[TN * kRow];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = wave / 2, wn = wave % 2;
  constexpr int kOutCols = (kEpilogue == kMfSwiglu) ? TN / 2 : TN;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * kOutCols;

  // global -> register staging: TM * 8 chunks of 16 bytes per slab, NC per thread
  constexpr int NC = WT * 2;
  int c_row[NC];
#pragma unroll
  for (int j = 0; j < NC; ++j) c_row[j] = (tid + 256 * j) / 8;
  const int c_k = (tid % 8) * 8;
  const bf16_t* a_src[NC];
  const bf16_t* w_src[NC];
  bool a_ok[NC], w_ok[NC];
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int m = m0 + c_row[j];
    a_ok[j] = m < M;
    a_src[j] = A + static_cast<int64_t>(a_ok[j] ? m : 0) * lda + c_k;
    int n;
    const bf16_t* base = W;
    if (kEpilogue == kMfSwiglu) {  // slab rows 0..63: gate rows n0..n0+63, rows 64..127: up rows of the same columns
      n = n0 + (c_row[j] % 64);
      if (c_row[j] >= 64) base = W2;
    } else {
      n = n0 + c_row[j];
    }
    w_ok[j] = n < N;
    w_src[j] = base + static_cast<int64_t>(w_ok[j] ? n : 0) * ldw + c_k;
  }

  f32x16 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  uint4 a_reg[PF][NC], w_reg[PF][NC];
  auto fetch = [&](uint4 (&a)[NC], uint4 (&w)[NC], int k0) {
    // Every lane issues every load (from the row's start where the values are not wanted; zeros are put in
    // their place at staging): with loads that are always issued the compiler can count them and wait for
    // the oldest slab only, so that the later ones stay on their way.
    const int koff = (k0 + c_k < K) ? k0 : -c_k;
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      a[j] = *reinterpret_cast<const uint4*>(a_src[j] + koff);
      w[j] = *reinterpret_cast<const uint4*>(w_src[j] + koff);
    }
  };
  auto stage = [&](const uint4 (&a)[NC], const uint4 (&w)[NC], int k0) {
    const bool k_ok = k0 + c_k < K;
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      const uint32_t ka = 0u - static_cast<uint32_t>(k_ok && a_ok[j]), kw = 0u - static_cast<uint32_t>(k_ok && w_ok[j]);   // all ones or zero
      *reinterpret_cast<uint4*>(&As[c_row[j] * kRow + c_k]) = make_uint4(a[j].x & ka, a[j].y & ka, a[j].z & ka, a[j].w & ka);
      *reinterpret_cast<uint4*>(&Ws[c_row[j] * kRow + c_k]) = make_uint4(w[j].x & kw, w[j].y & kw, w[j].z & kw, w[j].w & kw);
    }
  };

  // rows of the fragments this lane reads
  const int frag_row = lane % 32, frag_k = (lane / 32) * 8;
  int a_off[WT], w_off[WT];
#pragma unroll
  for (int i = 0; i < WT; ++i) {
    a_off[i] = (wm * 32 * WT + i * 32 + frag_row) * kRow + frag_k;
    // swiglu: tile 0 = gate rows of this wave's 32 columns, tile 1 = the up rows of the same columns
    w_off[i] = ((kEpilogue == kMfSwiglu) ? (i * 64 + wn * 32 + frag_row) : (wn * 32 * WT + i * 32 + frag_row)) * kRow + frag_k;
  }
  auto multiply = [&]() {
#pragma unroll
    for (int ks = 0; ks < TK; ks += 16) {
      bf16x8 a[WT], w[WT];
#pragma unroll
      for (int i = 0; i < WT; ++i) {
        a[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&As[a_off[i] + ks]));
        w[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Ws[w_off[i] + ks]));
      }
#pragma unroll
      for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], w[j], acc[i][j], 0, 0, 0);
    }
  };

#pragma unroll
  for (int p = 0; p < PF; ++p) fetch(a_reg[p], w_reg[p], p * TK);
  for (int k0 = 0; k0 < K; k0 += PF * TK) {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      if (k0 + p * TK < K) {    // uniform over the block
        __syncthreads();        // the previous slab has been read by every wave
        stage(a_reg[p], w_reg[p], k0 + p * TK);
        __syncthreads();
        fetch(a_reg[p], w_reg[p], k0 + (p + PF) * TK);
        multiply();
      }
    }
  }

  // epilogue
  const int col = lane % 32, row_base = (lane / 32) * 4;
#pragma unroll
  for (int i = 0; i < WT; ++i) {
#pragma unroll
    for (int j = 0; j < ((kEpilogue == kMfSwiglu) ? 1 : WT); ++j) {
      const int n = (kEpilogue == kMfSwiglu) ? n0 + wn * 32 + col : n0 + wn * 32 * WT + j * 32 + col;
      if (n >= N) continue;
      const float b = (bias && kEpilogue == kMfStore) ? bias[n] : 0.f;
      const int m_first = m0 + wm * 32 * WT + i * 32 + row_base;      // element e: row m_first + 8 * (e / 4) + e % 4
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
          const float g = acc[i][0][e];
          store_f32(dst, g / (1.f + __expf(-g)) * acc[i][WT - 1][e]);
        }
      }
    }
  }
}

template <int kEpilogue, typename TO>
static int launch_mfma(void* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw,
                       const float* bias, int M, int N, int K, hipStream_t stream) {
  // Big tiles (one slab ahead) when they fill the chip: about two blocks per compute unit, which hide one
  // another's waits. Small tiles (two slabs ahead) otherwise: few big tiles, each alone on its compute
  // unit, were slower here even with four slabs ahead.
  const int64_t big_blocks = static_cast<int64_t>((N + 127) / 128) * ((M + 127) / 128);
  if (kEpilogue == kMfSwiglu || big_blocks >= 512) {
    constexpr int cols = (kEpilogue == kMfSwiglu) ? 64 : 128;
    dim3 grid((N + cols - 1) / cols, (M + 127) / 128);
    gemm_mfma_kernel<kEpilogue, TO, 2, 1><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), ldo, static_cast<const bf16_t*>(A), lda,
                                                                     static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2),
                                                                     ldw, bias, M, N, K);
  } else {
    constexpr int kE = (kEpilogue == kMfSwiglu) ? kMfStore : kEpilogue;   // (never taken for swiglu)
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    gemm_mfma_kernel<kE, TO, 1, 2><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), ldo, static_cast<const bf16_t*>(A), lda,
                                                              static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2), ldw,
                                                              bias, M, N, K);
  }
  return check_launch("gemm_mfma");
}

}  // namespace alofa

using namespace alofa;

// bfloat16 A [M, K] and W [N, K] (W2 for the swiglu epilogue); K a multiple of 8, rows 16-byte
// aligned. Epilogues: 0 store (+ bias) as o_dtype, 1 add to the float residual, 2 swiglu.
extern "C" int alofa_gemm_mfma(void* out, int o_dtype, int64_t ldo, const void* A, int64_t lda, const void* W,
                               const void* W2, int64_t ldw, const float* bias, int M, int N, int K, int epilogue,
                               hipStream_t stream) {
  ALOFA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_mfma: M=%d N=%d K=%d must be positive", M, N, K);
  ALOFA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_mfma: K=%d, lda=%lld, ldw=%lld must be multiples of 8", K,
                static_cast<long long>(lda), static_cast<long long>(ldw));
  ALOFA_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(W2) % 16 == 0, "gemm_mfma: operands must be 16-byte aligned");
  ALOFA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_mfma: a leading dimension is shorter than its row");
  if (epilogue == kMfStore && o_dtype == kBF16)
    return launch_mfma<kMfStore, bf16_t>(out, ldo, A, lda, W, nullptr, ldw, bias, M, N, K, stream);
  if (epilogue == kMfStore && o_dtype == kF32)
    return launch_mfma<kMfStore, float>(out, ldo, A, lda, W, nullptr, ldw, bias, M, N, K, stream);
  if (epilogue == kMfResidual && o_dtype == kF32)
    return launch_mfma<kMfResidual, float>(out, ldo, A, lda, W, nullptr, ldw, nullptr, M, N, K, stream);
  if (epilogue == kMfSwiglu && o_dtype == kBF16) {
    ALOFA_REQUIRE(W2 != nullptr, "gemm_mfma: the swiglu epilogue needs the up matrix");
    return launch_mfma<kMfSwiglu, bf16_t>(out, ldo, A, lda, W, W2, ldw, nullptr, M, N, K, stream);
  }
  ALOFA_REQUIRE(false, "gemm_mfma: unsupported epilogue %d with out dtype %d", epilogue, o_dtype);
}
