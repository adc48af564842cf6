// Choosing a token from a row of float logits on the device: the first maximum
// (greedy), or a draw from softmax(logits / temperature) by inverse CDF with a
// uniform number the host supplies. The draw works in double: weights
// exp(x/T - max), summed in index order within a thread's contiguous range and
// then across threads in thread order, and the first index whose running sum
// exceeds u * total is taken (the last index if none does).
#include "common.h"

#include <float.h>

namespace alofa {

constexpr int kPickThreads = 1024;

__global__ void __launch_bounds__(kPickThreads) argmax_kernel(int32_t* __restrict__ out, const float* __restrict__ logits,
                                                              int64_t stride, int vocab) {
  __shared__ float best_v[kPickThreads / kWave];
  __shared__ int best_i[kPickThreads / kWave];
  const float* row = logits + static_cast<int64_t>(blockIdx.x) * stride;
  float bv = -FLT_MAX;
  int bi = vocab;  // "none yet": any real index is lower
  for (int i = threadIdx.x; i < vocab; i += kPickThreads) {
    const float v = row[i];
    if (v > bv) { bv = v; bi = i; }
  }
  // strictly larger wins; equal values keep the lower index
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (lane == 0) { best_v[wave] = bv; best_i[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kPickThreads / kWave; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
    out[blockIdx.x] = bi < vocab ? bi : 0;
  }
}

__global__ void __launch_bounds__(kPickThreads) sample_kernel(int32_t* __restrict__ out, const float* __restrict__ logits,
                                                              int64_t stride, int vocab,
                                                              const double* __restrict__ temperature,
                                                              const double* __restrict__ uniform) {
  __shared__ double part[kPickThreads];
  __shared__ double red[kPickThreads / kWave];
  __shared__ int found;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + static_cast<int64_t>(r) * stride;
  const double temp = temperature[r];
  const int chunk = (vocab + kPickThreads - 1) / kPickThreads;
  const int lo = tid * chunk, hi = (lo + chunk < vocab) ? lo + chunk : vocab;

  double m = -1.0e300;
  for (int i = lo; i < hi; ++i) m = fmax(m, static_cast<double>(row[i]) / temp);
  for (int off = kWave / 2; off > 0; off >>= 1) m = fmax(m, __shfl_xor(m, off, kWave));
  if (tid % kWave == 0) red[tid / kWave] = m;
  __syncthreads();
  for (int w = 0; w < kPickThreads / kWave; ++w) m = fmax(m, red[w]);

  double mine = 0;
  for (int i = lo; i < hi; ++i) mine += exp(static_cast<double>(row[i]) / temp - m);
  part[tid] = mine;
  if (tid == 0) found = vocab - 1;
  __syncthreads();
  // exclusive prefix over threads, in thread order (each thread adds up its predecessors)
  double before = 0, total = 0;
  for (int i = 0; i < kPickThreads; ++i) {
    if (i == tid) before = total;
    total += part[i];
  }
  const double target = uniform[r] * total;
  if (lo < hi && before <= target && target < before + mine) {
    double acc = before;
    int pick = hi - 1;
    for (int i = lo; i < hi; ++i) {
      acc += exp(static_cast<double>(row[i]) / temp - m);
      if (target < acc) { pick = i; break; }
    }
    atomicMin(&found, pick);
  }
  __syncthreads();
  if (tid == 0) out[r] = found;
}

}  // namespace alofa

using namespace alofa;

extern "C" int alofa_argmax(int32_t* out, const float* logits, int64_t stride, int rows, int vocab,
                            hipStream_t stream) {
  ALOFA_REQUIRE(rows > 0 && vocab > 0 && stride >= vocab, "argmax: rows=%d vocab=%d stride=%lld", rows, vocab, static_cast<long long>(stride));
  argmax_kernel<<<rows, kPickThreads, 0, stream>>>(out, logits, stride, vocab);
  return check_launch("argmax");
}

extern "C" int alofa_sample(int32_t* out, const float* logits, int64_t stride, int rows, int vocab,
                            const double* temperature, const double* uniform, hipStream_t stream) {
  ALOFA_REQUIRE(rows > 0 && vocab > 0 && stride >= vocab, "sample: rows=%d vocab=%d stride=%lld", rows, vocab, static_cast<long long>(stride));
  sample_kernel<<<rows, kPickThreads, 0, stream>>>(out, logits, stride, vocab, temperature, uniform);
  return check_launch("sample");
}
