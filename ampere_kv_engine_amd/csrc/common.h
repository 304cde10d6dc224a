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

// Per-request state of fixed size on the device: kSlotWords 32-bit words per slot.  This is the one definition for
// the kernels; the host's (cache/slots.py) is checked against it when the library is loaded (akv_slot_layout).
constexpr int kSlotWords = 8;
enum SlotWord : int {
  kSlotLength = 0,       // tokens held
  kSlotLastToken = 1,    // the token chosen last (-1: none yet)
  kSlotTemperature = 2,  // float bits
  kSlotSeedLow = 3,
  kSlotSeedHigh = 4,
  kSlotDraws = 5,        // draws made so far
  kSlotTaken = 6,        // whether a request holds the slot
};

// Blocks of one launch that hand sums to each other through memory do it in three steps.  (1) The sums are written
// with device-scope atomic stores (`publish`): such a store goes through to where every XCD sees it.  (2) The block
// ticks a counter with `arrive`: first a wait until the wave's memory counters are at zero - every store it has
// issued has been acknowledged -, then a device-scope read-modify-write; compiler-only fences on either side of both
// keep the compiler from moving a store below the wait, the tick above it, or a later load above the tick (the wait
// is an instruction, not a memory operation: by itself it orders nothing for the compiler).  (3) Whoever learns from
// the counter that the others have been there reads their sums with device-scope atomic loads (`collect`), which do
// not take a stale copy from a cache; they are issued after the tick has returned its value.  Nobody waits for
// anybody.
// Under the memory model alone the order would need the tick to be a release and an acquire at device scope, and
// this device pays for those with a write-back of the XCD's L2 before the tick and its invalidation after (measured
// with the tick written so: 28 -> 30 us and 43 -> 45 us for products of 128 rows whose k is cut over blocks, 20 ->
// 27 us for a decode product whose row tiles straddle blocks) - although not one of the bytes concerned ever lies
// in a cache that another XCD does not see.  What is relied on beyond the model is a fact of the hardware: a
// device-scope store that has been acknowledged is seen by every later device-scope load or read-modify-write,
// whichever XCD issues it.
__device__ __forceinline__ void publish(float* at, float value) {
  __hip_atomic_store(at, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float collect(const float* at) {
  return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned arrive(unsigned* counter) {
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0);       // every counter at zero: the wave's stores have arrived
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  const unsigned before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  return before;
}

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

namespace akv {

// What the host needs to know of the device it launches on to cut work into blocks: asked of the runtime once per
// device.  (The number of XCDs is not among a device's attributes: gfx950 parts have 8, each with an L2 of its own.)
struct DeviceFacts {
  int compute_units;
  size_t lds_bytes;     // LDS of a compute unit: the most a block can ask for
};
constexpr int kXcds = 8;

inline DeviceFacts device_facts() {
  static DeviceFacts known[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return DeviceFacts{256, 160 * 1024};
  if (known[device].compute_units == 0) {       // (two threads asking at once write the same values)
    int units = 0, lds = 0;
    if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0) units = 256;
    if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device) != hipSuccess || lds <= 0)
      lds = 160 * 1024;
    known[device] = DeviceFacts{units, static_cast<size_t>(lds)};
  }
  return known[device];
}

}  // namespace akv
