// Shared device helpers for the gfx950 kernels: storage types, wave-64 reductions, dtype dispatch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace akv {

constexpr int kWave = 64;

// bfloat16 as stored: the upper 16 bits of a float.  Conversion to float is exact; conversion from float
// rounds to nearest, ties to even, and keeps NaN a NaN.
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(static_cast<uint32_t>(x.bits) << 16); }

// (gfx950 converts in hardware - v_cvt_pk_bf16_f32, two values an instruction - which the compiler emits for a cast to
// its own bfloat type; in software the same rounding is seven instructions a value.)
__device__ __forceinline__ uint16_t bf16_bits(float x) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(x)); }

// Two values rounded and packed as they lie in memory: `low` in the lower half.
__device__ __forceinline__ uint32_t bf16_pair(float low, float high) {
  typedef __attribute__((ext_vector_type(2))) float float_pair;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16_pair_t;
  const float_pair both = {low, high};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(both, bf16_pair_t));
}

template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float x) { return bf16_t{bf16_bits(x)}; }

// The value x has after being stored as T and read back.
template <typename T> __device__ __forceinline__ float rounded(float x) { return to_float(from_float<T>(x)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch` holds one float per wave.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

enum DType : int { kF32 = 0, kBF16 = 1 };

}  // namespace akv

// Expands `body` with `T` bound to the storage type named by `code`; unknown codes return -1.
#define AKV_DISPATCH(code, T, ...)                      \
  do {                                                  \
    if ((code) == akv::kF32) {                          \
      using T = float;                                  \
      __VA_ARGS__;                                      \
    } else if ((code) == akv::kBF16) {                  \
      using T = akv::bf16_t;                            \
      __VA_ARGS__;                                      \
    } else {                                            \
      return -1;                                        \
    }                                                   \
  } while (0)

#define AKV_LAUNCH_STATUS() static_cast<int>(hipGetLastError())
