// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave and block reductions, and the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

namespace alofa {

typedef uint16_t bf16_t;  // bfloat16 carried as its 16 bits

constexpr int kWave = 64;  // CDNA wavefront

enum DType : int { kF32 = 0, kBF16 = 1 };

// ---- conversions -----------------------------------------------------------

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// two floats to a pair of bfloat16 (a in the low half), round to nearest even:
// the hardware conversion v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return static_cast<bf16_t>(pack_bf16x2(f, 0.f) & 0xffffu); }

template <typename T> __device__ __forceinline__ float load_f32(const T* p);
template <> __device__ __forceinline__ float load_f32<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }

template <typename T> __device__ __forceinline__ void store_f32(T* p, float v);
template <> __device__ __forceinline__ void store_f32<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// ---- reductions ------------------------------------------------------------

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a block of kThreads (a multiple of 64) in a fixed tree, so the
// result depends only on the inputs' places, never on timing. Every thread
// gets the total. `scratch` holds kThreads / 64 values.
template <typename T, int kThreads>
__device__ __forceinline__ T block_sum(T v, T* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  T total = scratch[0];
#pragma unroll
  for (int w = 1; w < kThreads / kWave; ++w) total += scratch[w];
  return total;
}

// ---- workspace ---------------------------------------------------------------
// Scratch for kernels whose blocks hand partial results to one another (the K split of the
// few-rows product): `tiles` for the partial results and zeroed counters, in uncached device memory, so that what one block wrote is what another
// reads, whichever die they run on, without flushing caches. The library allocates it once
// per process (alofa_workspace_init) and never frees it. Every kernel leaves its counters
// zero. Kernels that use it must not overlap on one GPU (one stream at a time).
struct Workspace {
  float* tiles;
  int64_t tile_floats;
  int* counters;
  int n_counters;
};
constexpr int kGemmCounters = 4096;   // counters the few-rows product may use
const Workspace& workspace();

// ---- error channel ---------------------------------------------------------

void set_error(const char* fmt, ...);
int check_launch(const char* what);

}  // namespace alofa

#define ALOFA_REQUIRE(cond, ...)          \
  do {                                    \
    if (!(cond)) {                        \
      alofa::set_error(__VA_ARGS__);      \
      return 1;                           \
    }                                     \
  } while (0)
