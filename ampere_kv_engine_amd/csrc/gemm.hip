// Matrix products y = x W^T for x [rows, k], W [out, k] (row-major, as checkpoints store them).
//
// `linear_tiled` is the plain path: float32 multiply-add on 64x64 output tiles staged through LDS, for any
// mix of float32 / bfloat16 operands and any sizes.  Every output element is one sum over k in ascending order
// inside fixed k-tiles, so a row's result does not depend on how many other rows the call carries.  It is the
// whole of the float32 path and the fallback for operand mixes the MFMA kernels do not take.

#include "common.h"
#include "api.h"

using namespace akv;

namespace {

constexpr int kTile = 64;   // output tile edge
constexpr int kDepth = 16;  // k-tile

template <typename TX, typename TW, typename TY>
__global__ __launch_bounds__(256) void linear_tiled_kernel(const TX* __restrict__ x, const TW* __restrict__ w,
                                                           TY* __restrict__ y, int rows, int outs, int k,
                                                           const float* __restrict__ bias) {
  __shared__ float xs[kDepth][kTile + 1];
  __shared__ float ws[kDepth][kTile + 1];
  const int row0 = blockIdx.y * kTile, out0 = blockIdx.x * kTile;
  const int tr = threadIdx.x / 16, tc = threadIdx.x % 16;  // 16 x 16 threads, each a 4 x 4 patch
  float acc[4][4] = {};
  for (int k0 = 0; k0 < k; k0 += kDepth) {
    // 64 x 16 elements of each operand, 4 per thread; out-of-range elements are zeros
    for (int e = threadIdx.x; e < kTile * kDepth; e += 256) {
      const int r = e / kDepth, c = e % kDepth;
      const bool in_k = k0 + c < k;
      xs[c][r] = (in_k && row0 + r < rows) ? to_float(x[static_cast<size_t>(row0 + r) * k + k0 + c]) : 0.f;
      ws[c][r] = (in_k && out0 + r < outs) ? to_float(w[static_cast<size_t>(out0 + r) * k + k0 + c]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < kDepth; ++c) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[c][tr * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[c][tc * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + tr * 4 + i;
    if (r >= rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int o = out0 + tc * 4 + j;
      if (o < outs) y[static_cast<size_t>(r) * outs + o] = from_float<TY>(bias != nullptr ? acc[i][j] + bias[o] : acc[i][j]);
    }
  }
}

template <typename TX, typename TW, typename TY>
int launch_tiled(const void* x, const void* w, void* y, int rows, int outs, int k, const float* bias, hipStream_t stream) {
  dim3 grid((outs + kTile - 1) / kTile, (rows + kTile - 1) / kTile);
  linear_tiled_kernel<TX, TW, TY><<<grid, 256, 0, stream>>>(static_cast<const TX*>(x), static_cast<const TW*>(w),
                                                            static_cast<TY*>(y), rows, outs, k, bias);
  return AKV_LAUNCH_STATUS();
}

}  // namespace

// `bias` [outs] float32 or null: added to a sum after its last product, before it is rounded to y's type.
extern "C" int akv_linear_tiled(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype, int rows,
                                int outs, int k, const float* bias, hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if (((rows + kTile - 1) / kTile) > 65535) return -2;
  const int code = x_dtype * 4 + w_dtype * 2 + y_dtype;
  switch (code) {
    case 0: return launch_tiled<float, float, float>(x, w, y, rows, outs, k, bias, stream);
    case 2: return launch_tiled<float, bf16_t, float>(x, w, y, rows, outs, k, bias, stream);
    case 4: return launch_tiled<bf16_t, float, float>(x, w, y, rows, outs, k, bias, stream);
    case 5: return launch_tiled<bf16_t, float, bf16_t>(x, w, y, rows, outs, k, bias, stream);
    case 6: return launch_tiled<bf16_t, bf16_t, float>(x, w, y, rows, outs, k, bias, stream);
    case 7: return launch_tiled<bf16_t, bf16_t, bf16_t>(x, w, y, rows, outs, k, bias, stream);
    default: return -1;
  }
}
