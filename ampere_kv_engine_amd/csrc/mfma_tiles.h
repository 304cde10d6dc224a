// Pieces shared by the bfloat16 matrix-product kernels: operand vector types, the 16 x 16 x 32 matrix-core
// instruction, the load of bytes that are used once, and the store of a 16 x 16 result tile.
#pragma once

#include "common.h"

namespace akv {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;  // 16 bytes of operand: 8 bfloat16 (a plain vector
                                                                 // type: the compiler keeps it in registers)

__device__ __forceinline__ floatx4 mfma16(uintx4 a, uintx4 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// A 16-byte read of data that is used once: it does not displace what others re-read from the caches.
__device__ __forceinline__ uintx4 load_once(const uintx4* p) { return __builtin_nontemporal_load(p); }

// Where tile (row_tile, kt) of a packed matrix lies, counted in tiles of 1 KB.  Plain: [row tile][k tile].  PAIRED (the
// gated feed-forward's matrix, whose row tiles come in pairs of gate and up rows that one wave always owns together):
// [pair][k tile][2] - the pair's two tiles of a k-tile lie side by side, so the wave streams ONE contiguous run of
// memory along k instead of two runs a whole row tile apart (measured at 2 x 12,288 x 4,096: 39 -> 34 us for the
// bare reads of a decode step's product).
template <bool PAIRED>
__host__ __device__ __forceinline__ size_t tile_index(int row_tile, int kt, int k_tiles) {
  return PAIRED ? (static_cast<size_t>(row_tile >> 1) * k_tiles + kt) * 2 + (row_tile & 1)
                : static_cast<size_t>(row_tile) * k_tiles + kt;
}

template <typename TY> __device__ __forceinline__ void store4(TY* p, floatx4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, floatx4 v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, floatx4 v) {
  uint2 packed;
  packed.x = bf16_pair(v[0], v[1]);
  packed.y = bf16_pair(v[2], v[3]);
  *reinterpret_cast<uint2*>(p) = packed;
}

// Lane (r = l % 16, g = l / 16) owns outputs [feature0 + g * 4 + i][token r] of a 16 x 16 tile.
template <typename TY>
__device__ __forceinline__ void store_tile(TY* y, floatx4 acc, int token, int feature, int rows, int outs) {
  if (token >= rows) return;
  TY* dst = y + static_cast<size_t>(token) * outs + feature;
  if (feature + 3 < outs && (outs & 3) == 0) {
    store4<TY>(dst, acc);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (feature + i < outs) dst[i] = from_float<TY>(acc[i]);
  }
}

// The tile's four values plus the bias of their features; `bias` [outs] may be null: then nothing is added.  (A product
// with a bias is x W^T + b formed in float32 and rounded once, as torch.nn.functional.linear forms it.)
__device__ __forceinline__ floatx4 plus_bias(floatx4 acc, const float* __restrict__ bias, int feature, int outs) {
  if (bias != nullptr) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (feature + i < outs) acc[i] += bias[feature + i];
  }
  return acc;
}

__device__ __forceinline__ floatx4 silu_times(floatx4 gate, floatx4 up) {
  floatx4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = gate[i] / (1.f + expf(-gate[i])) * up[i];
  return v;
}

}  // namespace akv
