// Choosing a token from a row of float logits on the device: the first maximum
// (greedy), or a draw from softmax(logits / temperature) by inverse CDF with a
// uniform number the host supplies. The draw works in double: weights
// exp(x/T - max), summed in index order within a thread's contiguous range and
// then across threads in thread order, and the first index whose running sum
// exceeds u * total is taken (the last index if none does).
#include "common.h"
#include "no_alloc.h"

#include <float.h>

#include <mutex>

namespace alofa {

constexpr int kPickThreads = 1024;

// Where a choice goes: out[r], and, when a store is given, store[store_index[r]] as well (the token
// of request slot store_index[r], which the next step's embedding reads without a trip to the host).
struct Choice {
  int32_t* out;
  int32_t* store;
  const int32_t* store_index;
  __device__ __forceinline__ void put(int r, int token) const {
    out[r] = token;
    if (store) store[store_index[r]] = token;
  }
};

__global__ void __launch_bounds__(kPickThreads) argmax_kernel(Choice choice, const float* __restrict__ logits,
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
    choice.put(blockIdx.x, bi < vocab ? bi : 0);
  }
}

// Two-stage form for long rows: kArgmaxChunks blocks per row each find the first
// maximum of a contiguous chunk, then one wave per row takes the first maximum of
// the chunks in chunk order (a lower chunk holds lower indices, so ties still go
// to the lowest index).
constexpr int kArgmaxChunks = 64;

__global__ void __launch_bounds__(256) argmax_chunk_kernel(float* __restrict__ part_v, int32_t* __restrict__ part_i,
                                                           const float* __restrict__ logits, int64_t stride, int vocab) {
  __shared__ float best_v[4];
  __shared__ int best_i[4];
  const int r = blockIdx.y, chunk = blockIdx.x;
  const int per = (vocab + kArgmaxChunks - 1) / kArgmaxChunks;
  const int lo = chunk * per, hi = (lo + per < vocab) ? lo + per : vocab;
  const float* row = logits + static_cast<int64_t>(r) * stride;
  float bv = -FLT_MAX;
  int bi = vocab;
  for (int i = lo + threadIdx.x; i < hi; i += 256) {
    const float v = row[i];
    if (v > bv) { bv = v; bi = i; }
  }
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if (threadIdx.x % kWave == 0) { best_v[threadIdx.x / kWave] = bv; best_i[threadIdx.x / kWave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
    part_v[r * kArgmaxChunks + chunk] = bv;
    part_i[r * kArgmaxChunks + chunk] = bi;
  }
}

__global__ void __launch_bounds__(kWave) argmax_final_kernel(Choice choice, const float* __restrict__ part_v,
                                                             const int32_t* __restrict__ part_i, int vocab) {
  const int r = blockIdx.x;
  float bv = part_v[r * kArgmaxChunks + threadIdx.x];
  int bi = part_i[r * kArgmaxChunks + threadIdx.x];
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if (threadIdx.x == 0) choice.put(r, bi < vocab ? bi : 0);
}

// The same last stage over any number of candidates per row (value and index each, indices ascending with the
// candidate's number or not): the highest value, the lowest index among equals. For candidates that the
// vocabulary product leaves instead of logits.
__global__ void __launch_bounds__(256) argmax_parts_kernel(Choice choice, const float* __restrict__ part_v,
                                                           const int32_t* __restrict__ part_i, int n_parts, int vocab) {
  __shared__ float best_v[4];
  __shared__ int best_i[4];
  const int r = blockIdx.x;
  float bv = -FLT_MAX;
  int bi = vocab;
  // (eight candidates' loads on their way together; compared in ascending order as one by one)
  const float* row_v = part_v + static_cast<int64_t>(r) * n_parts;
  const int32_t* row_i = part_i + static_cast<int64_t>(r) * n_parts;
  for (int p0 = threadIdx.x; p0 < n_parts; p0 += 8 * 256) {
    float vs[8];
    int is[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int p = min(p0 + 256 * u, n_parts - 1);
      vs[u] = row_v[p];
      is[u] = row_i[p];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (p0 + 256 * u < n_parts && (vs[u] > bv || (vs[u] == bv && is[u] < bi))) { bv = vs[u]; bi = is[u]; }
  }
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if (threadIdx.x % kWave == 0) { best_v[threadIdx.x / kWave] = bv; best_i[threadIdx.x / kWave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
    choice.put(r, bi < vocab ? bi : 0);
  }
}

__global__ void __launch_bounds__(kPickThreads) sample_kernel(Choice choice, const float* __restrict__ logits,
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
  if (tid == 0) choice.put(r, found);
}

}  // namespace alofa

using namespace alofa;

static int argmax_with(Choice choice, const float* logits, int64_t stride, int rows, int vocab, void* scratch, hipStream_t stream);

// scratch: rows * 64 floats followed by rows * 64 int32 for long rows (null: one block per row)
extern "C" int alofa_argmax(int32_t* out, const float* logits, int64_t stride, int rows, int vocab, void* scratch,
                            hipStream_t stream) {
  return argmax_with(Choice{out, nullptr, nullptr}, logits, stride, rows, vocab, scratch, stream);
}

// The same, and store[store_index[r]] = out[r] as well (store_index: rows int32 indices the caller has checked
// against the store's length).
extern "C" int alofa_argmax_to_store(int32_t* out, const float* logits, int64_t stride, int rows, int vocab, void* scratch,
                                     int32_t* store, const int32_t* store_index, hipStream_t stream) {
  ALOFA_REQUIRE(store != nullptr && store_index != nullptr, "argmax_to_store: store and store_index must be given");
  return argmax_with(Choice{out, store, store_index}, logits, stride, rows, vocab, scratch, stream);
}

static int argmax_with(Choice choice, const float* logits, int64_t stride, int rows, int vocab, void* scratch, hipStream_t stream) {
  ALOFA_REQUIRE(rows > 0 && vocab > 0 && stride >= vocab, "argmax: rows=%d vocab=%d stride=%lld", rows, vocab, static_cast<long long>(stride));
  if (scratch == nullptr) {
    argmax_kernel<<<rows, kPickThreads, 0, stream>>>(choice, logits, stride, vocab);
    return check_launch("argmax");
  }
  float* part_v = static_cast<float*>(scratch);
  int32_t* part_i = reinterpret_cast<int32_t*>(part_v + static_cast<int64_t>(rows) * kArgmaxChunks);
  argmax_chunk_kernel<<<dim3(kArgmaxChunks, rows), 256, 0, stream>>>(part_v, part_i, logits, stride, vocab);
  if (check_launch("argmax_chunk")) return 1;
  argmax_final_kernel<<<rows, kWave, 0, stream>>>(choice, part_v, part_i, vocab);
  return check_launch("argmax_final");
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// The partial maxima of alofa_argmax_no_alloc live in this array instead of a buffer the caller
// brings. In host code the array's name is only a stand-in: the memory is reached through the
// address that hipGetSymbolAddress gives, looked up once per device (every GPU holds a copy of its
// own) with that device current.
namespace alofa {

constexpr int64_t kNoAllocScratchBytes = static_cast<int64_t>(ALOFA_ARGMAX_NO_ALLOC_MAX_ROWS) * kArgmaxChunks * (sizeof(float) + sizeof(int32_t));
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_scratch_of_device[kMaxDevices];   // null until the first call on that device
static std::mutex g_scratch_mutex;

// the current device's copy of `scratch`, or null with the error set
static void* scratch_of_current_device() {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
    set_error("argmax_no_alloc: no usable current device: %s [device=%d]", hipGetErrorString(e), device);
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (g_scratch_of_device[device] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("argmax_no_alloc: the scratch array has no address on device %d: %s", device, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_of_device[device] = ptr;
  }
  return g_scratch_of_device[device];
}

}  // namespace alofa

extern "C" int alofa_argmax_no_alloc(int32_t* out, const float* logits, int64_t stride, int rows, int vocab, hipStream_t stream) {
  ALOFA_REQUIRE(out != nullptr && logits != nullptr, "argmax_no_alloc: out and logits must be given");
  ALOFA_REQUIRE(rows > 0 && vocab > 0 && stride >= vocab, "argmax_no_alloc: rows=%d vocab=%d stride=%lld", rows, vocab, static_cast<long long>(stride));
  ALOFA_REQUIRE(rows <= ALOFA_ARGMAX_NO_ALLOC_MAX_ROWS, "argmax_no_alloc: at most %d rows fit the built-in scratch [rows=%d]",
                ALOFA_ARGMAX_NO_ALLOC_MAX_ROWS, rows);
  void* ptr = scratch_of_current_device();
  if (ptr == nullptr) return 1;
  // every (row, chunk) cell that the second kernel reads is written by the first, so nothing
  // of an earlier call's contents has to be cleared
  float* part_v = static_cast<float*>(ptr);
  int32_t* part_i = reinterpret_cast<int32_t*>(part_v + static_cast<int64_t>(rows) * kArgmaxChunks);
  argmax_chunk_kernel<<<dim3(kArgmaxChunks, rows), 256, 0, stream>>>(part_v, part_i, logits, stride, vocab);
  if (check_launch("argmax_chunk")) return 1;
  argmax_final_kernel<<<rows, kWave, 0, stream>>>(Choice{out, nullptr, nullptr}, part_v, part_i, vocab);
  return check_launch("argmax_final");
}

// out[r] = the index of the highest of row r's n_parts candidates (part_v, part_i: [rows, n_parts]; an index of
// `vocab` or more stands for "none"), the lowest index among equal values; store and store_index both null or
// as for alofa_argmax_to_store.
extern "C" int alofa_argmax_parts(int32_t* out, int32_t* store, const int32_t* store_index, const float* part_v,
                                  const int32_t* part_i, int rows, int n_parts, int vocab, hipStream_t stream) {
  ALOFA_REQUIRE(out != nullptr && part_v != nullptr && part_i != nullptr && rows > 0 && n_parts > 0 && vocab > 0,
                "argmax_parts: rows=%d parts=%d vocab=%d", rows, n_parts, vocab);
  ALOFA_REQUIRE((store == nullptr) == (store_index == nullptr), "argmax_parts: a store goes with its index");
  argmax_parts_kernel<<<rows, 256, 0, stream>>>(Choice{out, store, store_index}, part_v, part_i, n_parts, vocab);
  return check_launch("argmax_parts");
}

// store and store_index: both null, or as for alofa_argmax_to_store
extern "C" int alofa_sample(int32_t* out, const float* logits, int64_t stride, int rows, int vocab,
                            const double* temperature, const double* uniform, int32_t* store, const int32_t* store_index,
                            hipStream_t stream) {
  ALOFA_REQUIRE(rows > 0 && vocab > 0 && stride >= vocab, "sample: rows=%d vocab=%d stride=%lld", rows, vocab, static_cast<long long>(stride));
  ALOFA_REQUIRE((store == nullptr) == (store_index == nullptr), "sample: store and store_index go together");
  sample_kernel<<<rows, kPickThreads, 0, stream>>>(Choice{out, store, store_index}, logits, stride, vocab, temperature, uniform);
  return check_launch("sample");
}
