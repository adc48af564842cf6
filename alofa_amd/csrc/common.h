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
// Sums and maxima over the 64 lanes of a wavefront ride on data-parallel-primitive moves between
// neighbouring lanes (no trip through LDS): a scan within each row of 16 lanes (shifts by 1, 2, 4, 8),
// then row 0's total into row 1 and row 2's into row 3, then the lower half's total into the upper half;
// lane 63 holds the result, which every lane reads. The order of the additions is fixed.

template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_move(float identity, float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(__float_as_uint(identity), __float_as_uint(v), kCtrl, kRowMask, 0xf, false));
}
template <int kCtrl, int kRowMask>
__device__ __forceinline__ double dpp_move(double identity, double v) {
  const uint64_t i = __builtin_bit_cast(uint64_t, identity), x = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = __builtin_amdgcn_update_dpp(static_cast<uint32_t>(i), static_cast<uint32_t>(x), kCtrl, kRowMask, 0xf, false);
  const uint32_t hi = __builtin_amdgcn_update_dpp(static_cast<uint32_t>(i >> 32), static_cast<uint32_t>(x >> 32), kCtrl, kRowMask, 0xf, false);
  return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);
}
__device__ __forceinline__ float read_lane(float v, int lane) {
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), lane));
}
__device__ __forceinline__ double read_lane(double v, int lane) {
  const uint64_t x = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(x), lane), hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(x >> 32), lane);
  return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);
}

constexpr int kRowShr1 = 0x111, kRowShr2 = 0x112, kRowShr4 = 0x114, kRowShr8 = 0x118, kRowBcast15 = 0x142, kRowBcast31 = 0x143;

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
  v += dpp_move<kRowShr1, 0xf>(T(0), v);
  v += dpp_move<kRowShr2, 0xf>(T(0), v);
  v += dpp_move<kRowShr4, 0xf>(T(0), v);
  v += dpp_move<kRowShr8, 0xf>(T(0), v);
  v += dpp_move<kRowBcast15, 0xa>(T(0), v);
  v += dpp_move<kRowBcast31, 0xc>(T(0), v);
  return read_lane(v, 63);
}

__device__ __forceinline__ float wave_max(float v) {
  constexpr float lowest = -3.402823466e+38f;
  v = fmaxf(v, dpp_move<kRowShr1, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<kRowShr2, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<kRowShr4, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<kRowShr8, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<kRowBcast15, 0xa>(lowest, v));
  v = fmaxf(v, dpp_move<kRowBcast31, 0xc>(lowest, v));
  return read_lane(v, 63);
}

// The four lanes l, l ^ 16, l ^ 32, l ^ 48 (one of each row of 16) meet: the rows are swapped in pairs,
// then the halves of the wavefront, by the lane-swap instructions; every lane gets the result.
__device__ __forceinline__ float rows_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// v of lane l ^ 1, l ^ 2 (within a quad of lanes) and l ^ 8 (within a row of 16), without LDS
__device__ __forceinline__ float lane_xor1(float v) { return dpp_move<0xB1, 0xf>(0.f, v); }   // quad_perm [1,0,3,2]
__device__ __forceinline__ float lane_xor2(float v) { return dpp_move<0x4E, 0xf>(0.f, v); }   // quad_perm [2,3,0,1]
__device__ __forceinline__ float lane_xor8(float v) { return dpp_move<0x128, 0xf>(0.f, v); }  // row_ror:8

// What this wavefront's lanes wrote to LDS is seen by its other lanes afterwards (LDS serves a
// wavefront's accesses in program order; the fences keep the compiler from moving them).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
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

// Compute units of the current device (asked once).
int compute_units();

// ---- error channel ---------------------------------------------------------

void set_error(const char* fmt, ...);
int check_launch(const char* what);

}  // namespace alofa

// (sampling.hip) the last stage of an argmax over candidates that another kernel left
extern "C" int alofa_argmax_parts(int32_t* out, int32_t* store, const int32_t* store_index, const float* part_v,
                                  const int32_t* part_i, int rows, int n_parts, int vocab, hipStream_t stream);


#define ALOFA_REQUIRE(cond, ...)          \
  do {                                    \
    if (!(cond)) {                        \
      alofa::set_error(__VA_ARGS__);      \
      return 1;                           \
    }                                     \
  } while (0)
