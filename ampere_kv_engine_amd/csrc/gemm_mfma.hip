// bfloat16 matrix products y = x W^T on the matrix cores (v_mfma_f32_16x16x32_bf16), float32 accumulation.
//
// W is not read row-major.  At load time it is packed into tiles of 16 output rows x 32 k, 1 KB each, stored
// [row_tile][k_tile][lane][8]: lane l of a wave holds row l % 16, k = (l / 16) * 8 .. + 8 of the tile, which is
// exactly the MFMA's A operand.  One global_load_dwordx4 per lane then brings a whole tile as 1 KB of consecutive
// bytes, and a wave that walks along k streams one contiguous region of memory - what HBM likes best.  Rows and k
// beyond the matrix are zero in the packing.
//
//   linear_skinny  rows <= 64 (decode): every wave streams its own tiles once; the few activations come from
//                  cache; k is split over the waves of a block and summed through LDS in a fixed order.
//   linear_wide    rows  > 64 (prefill): 128 x 128 output tiles per block, activations staged through LDS,
//                  weights straight from the packed layout into the A operand.
// In both, a row of x meets the weights in the same k order whatever else is in the batch.
//
// GATED variants compute a gated feed-forward's first half in one pass: the packed matrix alternates a tile of 16 gate
// rows with the tile of the 16 up rows of the same features, a wave always owns such pairs, and what it stores is
// silu(gate) * up, taken from the float32 accumulators - the stacked product never goes to memory.

#include <mutex>

#include "common.h"
#include "mfma_tiles.h"
#include "api.h"

using namespace akv;

// Where akv_linear_packed_static lays out its activations: device memory that exists from the moment the library is
// loaded until the process ends, on every GPU the library runs on, so that entry point never has to ask for any.
// In host code this name is only a handle for hipGetSymbolAddress; kernels are given the address that call returns.
constexpr size_t kStaticRowsBytes = 64 * 32768 * sizeof(uint16_t);   // 64 rows of 32,768 bfloat16: 4 MiB
static __device__ __align__(256) unsigned char scratch[kStaticRowsBytes];

namespace {

// ---- rows <= 16 * MT --------------------------------------------------------------------------------------------
// A wave owns RT consecutive row tiles and a part of k.  With more than 16 rows of x the activation operands weigh
// more than the weights (MT operands per weight tile); giving a wave RT row tiles lets each of them serve RT weight
// tiles, so the traffic from the caches stays near the traffic from memory.
// whether every wave of a block gets LDS for its own accumulators in the sum over the parts of k (8 waves, <= 64 KB)
template <int MT, int RT> constexpr bool kSkinnyOwnSets = RT * MT <= 8;
// k-tiles per group of loads: 8 weight tiles (8 KB) per group and wave - fewer where the activations' operands of a
// group (MT per k-tile) would not fit the registers beside them
template <int MT, int RT> constexpr int kSkinnyGroup = (RT == 1 && MT >= 3) ? 4 : 8 / RT;

// NORMED (a few rows): x is not read.  The rows are the residual sum `stream_in` (+ `delta`) normed as the norm
// kernel norms them - x * rsqrt(mean(x^2) + eps), rounded, times the weight, rounded - by every block for itself into
// LDS, while its first weights are on their way; block 0 also writes the new residual sum to `stream_out` (another
// buffer: the other blocks still read the old one).  That spares the step the norm's own launch.
struct NormIn {
  const float* stream_in;   // [rows, k]
  const bf16_t* delta;      // [rows, k] or null
  const float* weight;      // [k]
  float* stream_out;        // [rows, k], not stream_in
  float eps;
  int red_floats;           // floats of `red` before the rows in LDS
};

template <int MT, int RT, typename TY, bool GATED, bool NORMED = false>
__global__ __launch_bounds__(512) void linear_skinny_kernel(const bf16_t* __restrict__ x, const uintx4* __restrict__ wp,
                                                            TY* __restrict__ y, int rows, int outs, int k,
                                                            int k_tiles, int n_tiles, int k_split, int x_packed,
                                                            const NormIn norm, const float* __restrict__ bias) {
  constexpr int U = kSkinnyGroup<MT, RT>;  // k-tiles per group; two groups are in flight
  extern __shared__ float red[];  // [wave, or group of waves with the same row tiles][RT][MT][4][64]
  const int lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in every lane: keeps addresses scalar
  const int r = lane & 15, g = lane >> 4;
  const int row_tile = (blockIdx.x * (waves / k_split) + wave / k_split) * RT;
  const int part = wave % k_split;
  const int per_part = (k_tiles + k_split - 1) / k_split;
  const int kt0 = part * per_part, kt1 = min(k_tiles, kt0 + per_part);
  floatx4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bool works = row_tile < n_tiles && kt0 < kt1;
  // NORMED: the first group of weights is asked for before the rows are normed (every thread of the block takes part in
  // that, also those of waves without work), and handed to the loop below.
  constexpr int UN = NORMED ? U : 1;
  uintx4 early[NORMED ? RT : 1][UN];
  if constexpr (NORMED) {
    const uintx4 none = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int u = 0; u < U; ++u)
        early[rt][u] = (works && kt0 + u < kt1 && row_tile + rt < n_tiles)
                           ? load_once(wp + tile_index<GATED>(row_tile + rt, kt0 + u, k_tiles) * 64 + lane) : none;
    uint16_t* rows_lds = reinterpret_cast<uint16_t*>(red + norm.red_floats);
    // the waves share the rows: waves / rows of them take a row, each its own stride of the row's pieces of 8
    const int waves_per_row = max(1, waves / rows);
    const int row = wave / waves_per_row, part = wave % waves_per_row;
    const bool has_row = row < rows;
    const float* from = norm.stream_in + static_cast<size_t>(has_row ? row : 0) * k;
    const bf16_t* add = norm.delta != nullptr ? norm.delta + static_cast<size_t>(has_row ? row : 0) * k : nullptr;
    auto eight = [&](int i, float (&v)[8]) {
      const float4 lo = *reinterpret_cast<const float4*>(from + i), hi = *reinterpret_cast<const float4*>(from + i + 4);
      v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
      if (add != nullptr) {
        const uintx4 d = *reinterpret_cast<const uintx4*>(add + i);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          v[2 * w] += __uint_as_float(d[w] << 16);
          v[2 * w + 1] += __uint_as_float(d[w] & 0xffff0000u);
        }
      }
    };
    const int first = (part * 64 + lane) * 8, stride = waves_per_row * 64 * 8;
    float squares = 0.f;
    if (has_row) {
      for (int i = first; i < k; i += stride) {
        float v[8];
        eight(i, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) squares += v[e] * v[e];
      }
    }
    squares = wave_sum(squares);
    if (lane == 0) red[wave] = squares;
    __syncthreads();
    if (has_row) {
      float total = 0.f;
      for (int p = 0; p < waves_per_row; ++p) total += red[row * waves_per_row + p];  // the same order in every wave
      const float scale = rsqrtf(total / static_cast<float>(k) + norm.eps);
      for (int i = first; i < k; i += stride) {  // (the row comes from the caches the second time)
        float v[8];
        eight(i, v);
        if (blockIdx.x == 0) {
          float* to = norm.stream_out + static_cast<size_t>(row) * k + i;
          *reinterpret_cast<float4*>(to) = make_float4(v[0], v[1], v[2], v[3]);
          *reinterpret_cast<float4*>(to + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
        const float4 g0 = *reinterpret_cast<const float4*>(norm.weight + i), g1 = *reinterpret_cast<const float4*>(norm.weight + i + 4);
        const float gain[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        uintx4 packed;
#pragma unroll
        for (int w = 0; w < 4; ++w)
          packed[w] = bf16_pair(rounded<bf16_t>(v[2 * w] * scale) * gain[2 * w], rounded<bf16_t>(v[2 * w + 1] * scale) * gain[2 * w + 1]);
        *reinterpret_cast<uintx4*>(rows_lds + static_cast<size_t>(row) * k + i) = packed;
      }
    }
    __syncthreads();  // the rows are in LDS; `red` is free again
  }
  if (works) {
    // Addresses: a scalar base per wave plus a 32-bit lane offset, so that a load is one instruction.
    // bytes from the wave's first row tile to its rt-th, and from a k-tile to the next (a gated pair lies side by side)
    const size_t w_tile_bytes = static_cast<size_t>(k_tiles) * 1024;
    auto w_of = [&](int rt) { return GATED ? (rt >> 1) * 2 * w_tile_bytes + (rt & 1) * 1024 : rt * w_tile_bytes; };
    constexpr uint32_t kStep = GATED ? 2048u : 1024u;
    const char* w_wave = reinterpret_cast<const char*>(wp) + tile_index<GATED>(row_tile, 0, k_tiles) * 1024;
    const uint32_t w_lane = lane * 16u;
    const char* x_bytes = reinterpret_cast<const char*>(x);
    const uint32_t x_step = x_packed ? 1024u : 64u;  // bytes from a k-tile's operand to the next
    uint32_t x_lane[MT];
    bool x_row[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      x_row[mt] = mt * 16 + r < rows;
      // row-major x: row mt * 16 + r, 16 bytes at k = g * 8 of the k-tile.  Packed x ([row tile][k / 8][16 rows][8]):
      // the k-tile's operand is 1 KB of consecutive bytes, lane after lane, as the weights' is.
      x_lane[mt] = x_packed ? static_cast<uint32_t>(mt) * static_cast<uint32_t>(k) * 32u + lane * 16u
                            : static_cast<uint32_t>(mt * 16 + r) * static_cast<uint32_t>(k) * 2u + g * 16u;
    }
    const bool ragged = (k & 31) != 0;  // the last k-tile reaches beyond x's row
    const uintx4 zero = {0u, 0u, 0u, 0u};
    // Two sets of operand registers: while the matrix cores work on one group of U k-tiles, the loads of the next
    // group are already on their way.  Weights are read once and never again: their loads are marked nontemporal,
    // which leaves the caches to the activations that every wave reads.
    uintx4 a0[RT][U], a1[RT][U], b0[MT][U], b1[MT][U];
    auto fetch = [&](int kt, uintx4 (&a)[RT][U], uintx4 (&b)[MT][U]) {
      const char* w_at = w_wave + static_cast<size_t>(kt) * kStep;
      const char* x_at = x_bytes + static_cast<size_t>(kt) * x_step;
      if (kt + U <= kt1 && row_tile + RT <= n_tiles) {  // the whole group exists: no test per load
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int u = 0; u < U; ++u)
            a[rt][u] = load_once(reinterpret_cast<const uintx4*>(w_at + w_of(rt) + w_lane + u * kStep));
      } else {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int u = 0; u < U; ++u)
            a[rt][u] = (kt + u < kt1 && row_tile + rt < n_tiles)
                           ? load_once(reinterpret_cast<const uintx4*>(w_at + w_of(rt) + w_lane + u * kStep)) : zero;
      }
      if constexpr (NORMED) {  // the rows lie in LDS, normed: lane (r, g) reads row r, 16 bytes at k = g * 8 of the k-tile
        const char* rows_lds = reinterpret_cast<const char*>(red + norm.red_floats);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const bool inside = !ragged || (kt + u) * 32 + g * 8 < k;
            b[mt][u] = (kt + u < kt1 && x_row[mt] && inside)
                           ? *reinterpret_cast<const uintx4*>(rows_lds + (static_cast<size_t>(mt * 16 + r) * k + (kt + u) * 32 + g * 8) * 2)
                           : zero;
          }
      } else if (kt + U <= kt1 && !ragged) {  // one test per row tile of x instead of one per load
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
          for (int u = 0; u < U; ++u) b[mt][u] = zero;
          if (x_row[mt]) {
#pragma unroll
            for (int u = 0; u < U; ++u) b[mt][u] = *reinterpret_cast<const uintx4*>(x_at + x_lane[mt] + u * x_step);
          }
        }
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const bool inside = !ragged || (kt + u) * 32 + g * 8 < k;
            b[mt][u] = (kt + u < kt1 && x_row[mt] && inside)
                           ? *reinterpret_cast<const uintx4*>(x_at + x_lane[mt] + u * x_step) : zero;
          }
      }
    };
    auto multiply = [&](const uintx4 (&a)[RT][U], const uintx4 (&b)[MT][U]) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = mfma16(a[rt][u], b[mt][u], acc[rt][mt]);
    };
    fetch(kt0, a0, b0);
    if constexpr (NORMED) {  // (the weights of the first group were asked for before the rows were normed)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int u = 0; u < U; ++u) a0[rt][u] = early[rt][u];
    }
    for (int kt = kt0; kt < kt1; kt += 2 * U) {
      fetch(kt + U, a1, b1);      // beyond kt1 this fills zeros
      multiply(a0, b0);
      fetch(kt + 2 * U, a0, b0);
      multiply(a1, b1);
    }
  }
  if (k_split > 1) {
    // The parts of k are summed through LDS in a fixed order: part 0 + part 1 + part 2 ...  Where a set of
    // accumulators per wave fits, every wave writes its own and the wave of part 0 adds them up after one barrier;
    // otherwise one set per group of waves that share their row tiles is passed from part to part.
    constexpr int kSet = RT * MT * 4 * 64;  // floats of one wave's accumulators
    if constexpr (kSkinnyOwnSets<MT, RT>) {
      float* mine = red + static_cast<size_t>(wave) * kSet;
      if (part != 0) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[((rt * MT + mt) * 4 + i) * 64 + lane] = acc[rt][mt][i];
      }
      __syncthreads();
      if (part != 0) return;
      for (int other = 1; other < k_split; ++other) {
        const float* theirs = mine + static_cast<size_t>(other) * kSet;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[rt][mt][i] += theirs[((rt * MT + mt) * 4 + i) * 64 + lane];
      }
    } else {
      float* mine = red + static_cast<size_t>(wave / k_split) * kSet;
      for (int turn = 0; turn < k_split; ++turn) {
        if (part == turn) {
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                float* slot = mine + ((rt * MT + mt) * 4 + i) * 64 + lane;
                *slot = turn == 0 ? acc[rt][mt][i] : *slot + acc[rt][mt][i];
              }
        }
        __syncthreads();
      }
      if (part != 0) return;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[rt][mt][i] = mine[((rt * MT + mt) * 4 + i) * 64 + lane];
    }
  }
  if constexpr (GATED) {
    static_assert(RT % 2 == 0, "a wave must own gate and up tiles in pairs");
#pragma unroll
    for (int rt = 0; rt < RT; rt += 2)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        if (row_tile + rt < n_tiles)
          store_tile<TY>(y, silu_times(acc[rt][mt], acc[rt + 1][mt]), mt * 16 + r, ((row_tile + rt) >> 1) * 16 + g * 4,
                         rows, outs);
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        if (row_tile + rt < n_tiles)
          store_tile<TY>(y, plus_bias(acc[rt][mt], bias, (row_tile + rt) * 16 + g * 4, outs), mt * 16 + r,
                         (row_tile + rt) * 16 + g * 4, rows, outs);
  }
}

template <int MT, int RT, typename TY, bool GATED, bool NORMED = false>
int launch_skinny(const void* x, const void* wp, void* y, int rows, int outs, int k, int k_tiles, int n_tiles,
                  int x_packed, hipStream_t stream, const float* bias = nullptr, NormIn norm = NormIn{}) {
  // Enough waves to keep every CU's memory pipe full: k is split over the waves of a block when there are few row
  // tiles - down to short parts of k while the waves are very few, and further only while a wave keeps enough k-tiles
  // for two rounds of its double-buffered loop (measured: 1,536 waves of 32 k-tiles beat 3,072 of 16).
  constexpr int U = kSkinnyGroup<MT, RT>;
  const int wave_rows = (n_tiles + RT - 1) / RT;
  int k_split = 1;
  while (k_split < 8) {
    const int waves_now = wave_rows * k_split, part_after = k_tiles / (k_split * 2);
    if (!((waves_now < 1536 && part_after >= 4) || (waves_now < 2048 && part_after >= 4 * U))) break;
    k_split *= 2;
  }
  const int waves = k_split == 8 ? 8 : 4;
  const int rows_per_block = waves / k_split;
  const int blocks = (wave_rows + rows_per_block - 1) / rows_per_block;
  const size_t sets = kSkinnyOwnSets<MT, RT> ? waves : rows_per_block;
  size_t lds = k_split > 1 ? sets * RT * MT * 4 * 64 * sizeof(float) : 0;
  if constexpr (NORMED) {  // room for the block's sums, then the normed rows
    lds = lds < 64 ? 64 : lds;
    norm.red_floats = static_cast<int>(lds / sizeof(float));
    lds += static_cast<size_t>(rows) * k * 2;
    if (lds > 64 * 1024) return -2;
  }
  linear_skinny_kernel<MT, RT, TY, GATED, NORMED><<<blocks, waves * 64, lds, stream>>>(
      static_cast<const bf16_t*>(x), static_cast<const uintx4*>(wp), static_cast<TY*>(y), rows, outs, k, k_tiles,
      n_tiles, k_split, x_packed, norm, GATED ? nullptr : bias);
  return AKV_LAUNCH_STATUS();
}

template <typename TY, bool GATED>
int dispatch_skinny(const void* x, const void* wp, void* y, int rows, int outs, int k, int k_tiles, int n_tiles,
                    int x_packed, hipStream_t stream, const float* bias) {
  switch ((rows + 15) / 16) {
    case 1:
      // two row tiles per wave halve the activation loads per weight byte; that pays with several rows of x and
      // enough row tiles that the waves stay many (measured at 384 row tiles: 12.7 -> 11.5 us at 8 rows)
      if (GATED || (rows >= 4 && n_tiles >= 384 && n_tiles < 2048))
        return launch_skinny<1, 2, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
      return launch_skinny<1, GATED ? 2 : 1, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
    // Several tiles of x rows.  Two tiles: a wave takes 2 row tiles of the weights, or 1 where there are so few that
    // the blocks would not even cover the compute units (4,096 outputs: 15.6 -> 13.1 us at k = 4,096).  Three and
    // four: 4 row tiles where that still leaves a thousand waves (the gated product is measured better with 2 up to
    // 2,048 row tiles: 68.7 -> 51.8 us at 64 rows), 2 otherwise.
    case 2:
      if (!GATED && n_tiles <= 256)
        return launch_skinny<2, GATED ? 2 : 1, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
      return launch_skinny<2, 2, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
    case 3:
      if (!GATED && n_tiles <= 256)
        return launch_skinny<3, GATED ? 2 : 1, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
      return n_tiles >= (GATED ? 2048 : 512)
                 ? launch_skinny<3, 4, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias)
                 : launch_skinny<3, 2, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
    case 4:
      if (!GATED && n_tiles <= 256)
        return launch_skinny<4, GATED ? 2 : 1, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
      return n_tiles >= (GATED ? 2048 : 512)
                 ? launch_skinny<4, 4, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias)
                 : launch_skinny<4, 2, TY, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
    default: return -2;
  }
}

// ---- rows > 64 ----------------------------------------------------------------------------------------------------
// Block: 256 threads = 2 x 2 waves; block tile 256 tokens x 128 features; wave tile 128 tokens x 64 features
// = 8 x 4 MFMA tiles (128 accumulator registers).  Per stage of 64 k the block's activations [256 tokens][64 k] go
// through LDS, double-buffered, laid out [k chunk of 8][token] with the token index XOR-swizzled by the chunk so
// that both the staging writes (8 chunks of one token) and the operand reads (16 tokens of one chunk) are free of
// bank conflicts.  Weights come from the packed layout straight into A operands, one k-tile ahead of their use.
// Blocks are numbered so that the blocks sharing a band of 128 weight rows run on the same XCD (one L2 each: the
// band is fetched from memory once), while XCDs work on different bands.
constexpr int kWideN = 128, kWideK = 64;

// MW: token tiles per wave (8: 256 tokens per block; 4: 128 tokens per block, for products with few weight rows,
// which would otherwise leave compute units without a block).
template <typename TY, int MW, bool GATED>
__global__ __launch_bounds__(256, 2) void linear_wide_kernel(const bf16_t* __restrict__ x, const uintx4* __restrict__ wp,
                                                          TY* __restrict__ y, int rows, int outs, int k, int k_tiles,
                                                          int n_tiles, int n_blocks, int m_blocks,
                                                          const float* __restrict__ bias) {
  constexpr int kWideM = 32 * MW;  // tokens per block
  __shared__ uintx4 xs[2][kWideK / 8][kWideM];  // 2 stages x 8 chunks x tokens x 16 B (64 KB for 256 tokens)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  // block -> (band of weight rows, block of tokens): consecutive blocks of one XCD share the band
  const int xcd = blockIdx.x % kXcds, turn = blockIdx.x / kXcds;
  const int n_block = (turn / m_blocks) * kXcds + xcd, m_block = turn % m_blocks;
  if (n_block >= n_blocks) return;
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int token0 = m_block * kWideM, tile0 = n_block * (kWideN / 16) + wave_n * 4;
  const uintx4 zero = {0u, 0u, 0u, 0u};
  const int stages = (k_tiles + 1) / 2;

  floatx4 acc[4][MW];  // [feature tile][token tile]
#pragma unroll
  for (int n = 0; n < 4; ++n)
#pragma unroll
    for (int m = 0; m < MW; ++m) acc[n][m] = floatx4{0.f, 0.f, 0.f, 0.f};

  // staging: a thread moves 8 chunks of 16 B per stage; chunk c = e % 8 of token e / 8, so that 8 consecutive threads
  // read 128 consecutive bytes of one row of x.
  // No load of the loop stands behind a test: tokens beyond the last, k beyond the matrix and stages beyond the last
  // are asked for at the nearest address that exists, and what has to count as zero is zeroed when it is written to
  // LDS (weights beyond the matrix meet such zeros, or feed sums that are never stored).  With a test per load the
  // compiler cannot tell how many younger loads stand between a load and its use, and waits for all of them - those
  // it has just issued for the next stage included.
  const char* x_bytes = reinterpret_cast<const char*>(x);
  constexpr int PX = MW;  // 16-byte chunks a thread stages: tokens * 8 / 256
  uint32_t x_at[PX];
  bool x_row[PX];
#pragma unroll
  for (int p = 0; p < PX; ++p) {
    const int e = p * 256 + threadIdx.x, token = token0 + e / 8;
    x_row[p] = token < rows;
    x_at[p] = static_cast<uint32_t>(min(token, rows - 1)) * static_cast<uint32_t>(k) * 2u;
  }
  auto fetch = [&](int stage, uintx4 (&moving)[PX], unsigned& exists) {
    exists = 0u;
#pragma unroll
    for (int p = 0; p < PX; ++p) {
      const int e = p * 256 + threadIdx.x;
      const int col = stage * kWideK + (e % 8) * 8;
      exists |= (x_row[p] && col < k) ? 1u << p : 0u;
      moving[p] = *reinterpret_cast<const uintx4*>(x_bytes + x_at[p] + static_cast<uint32_t>(min(col, k - 8)) * 2u);
    }
  };
  auto stash = [&](int buffer, const uintx4 (&moving)[PX], unsigned exists) {
#pragma unroll
    for (int p = 0; p < PX; ++p) {
      const int e = p * 256 + threadIdx.x, c = e % 8, t = e / 8;
      xs[buffer][c][t ^ (c << 1)] = (exists >> p & 1u) ? moving[p] : zero;
    }
  };
  // weights: the wave's 4 row tiles of one k-tile
  const char* w_bytes = reinterpret_cast<const char*>(wp);
  auto weights = [&](int kt, uintx4 (&a)[4]) {
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const char* at = w_bytes + tile_index<GATED>(min(tile0 + n, n_tiles - 1), min(kt, k_tiles - 1), k_tiles) * 1024;
      a[n] = *reinterpret_cast<const uintx4*>(at + lane * 16u);
    }
  };
  auto multiply = [&](int buffer, int half, const uintx4 (&a)[4]) {
    uintx4 b[MW];
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      const int c = half * 4 + g, t = wave_m * (16 * MW) + m * 16 + r;
      b[m] = xs[buffer][c][t ^ (c << 1)];
    }
#pragma unroll
    for (int m = 0; m < MW; ++m)
#pragma unroll
      for (int n = 0; n < 4; ++n) acc[n][m] = mfma16(a[n], b[m], acc[n][m]);
    // Order for the instruction scheduler: two operand reads from LDS go out first, then every group of 4 matrix
    // instructions is followed by the read of the operand two groups ahead, so that the matrix pipe does not wait for
    // LDS (left alone, the scheduler puts every read right before its use).
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int m = 0; m < MW - 2; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
  };

  // (the fences: left alone, the compiler moves the loads behind the products that were to hide them, and the zeroing
  // of what has arrived up to where it waits for loads that were meant to have a stage's time)
  if constexpr (MW <= 4) {
    // Registers allow two sets of everything: the weights of a whole stage (two k-tiles) are fetched one stage ahead,
    // the activations two stages ahead (they wait in registers for one stage, then go to the LDS buffer that the
    // stage before has just finished reading).
    uintx4 a0[2][4], a1[2][4], m0[PX], m1[PX];
    unsigned e0, e1;
    auto run_stage = [&](int stage, const uintx4 (&cur)[2][4], uintx4 (&next)[2][4], uintx4 (&arriving)[PX],
                         unsigned& arriving_exists, const uintx4 (&arrived)[PX], unsigned arrived_exists) {
      const int buffer = stage & 1;
      fetch(stage + 2, arriving, arriving_exists);
      weights(stage * 2 + 2, next[0]);
      weights(stage * 2 + 3, next[1]);
      __builtin_amdgcn_sched_barrier(0);
      multiply(buffer, 0, cur[0]);
      multiply(buffer, 1, cur[1]);
      __builtin_amdgcn_sched_barrier(0);
      stash(buffer ^ 1, arrived, arrived_exists);
      __syncthreads();
    };
    fetch(0, m0, e0);
    stash(0, m0, e0);
    fetch(1, m1, e1);
    weights(0, a0[0]);
    weights(1, a0[1]);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    int stage = 0;
    for (; stage + 2 <= stages; stage += 2) {
      run_stage(stage, a0, a1, m0, e0, m1, e1);
      run_stage(stage + 1, a1, a0, m1, e1, m0, e0);
    }
    if (stage < stages) run_stage(stage, a0, a1, m0, e0, m1, e1);
  } else {
    // weights are fetched one k-tile ahead, activations one stage ahead
    uintx4 a0[4], a1[4], moving[PX];
    unsigned exists;
    fetch(0, moving, exists);
    stash(0, moving, exists);
    weights(0, a0);
    __syncthreads();
    for (int stage = 0; stage < stages; ++stage) {
      const int buffer = stage & 1;
      fetch(stage + 1, moving, exists);
      weights(stage * 2 + 1, a1);
      __builtin_amdgcn_sched_barrier(0);
      multiply(buffer, 0, a0);
      __builtin_amdgcn_sched_barrier(0);
      weights(stage * 2 + 2, a0);
      __builtin_amdgcn_sched_barrier(0);
      multiply(buffer, 1, a1);
      __builtin_amdgcn_sched_barrier(0);
      stash(buffer ^ 1, moving, exists);
      __syncthreads();
    }
  }
  if constexpr (GATED) {
#pragma unroll
    for (int n = 0; n < 4; n += 2)
#pragma unroll
      for (int m = 0; m < MW; ++m)
        store_tile<TY>(y, silu_times(acc[n][m], acc[n + 1][m]), token0 + wave_m * (16 * MW) + m * 16 + r,
                       ((tile0 + n) >> 1) * 16 + g * 4, rows, outs);
  } else {
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int m = 0; m < MW; ++m)
        store_tile<TY>(y, plus_bias(acc[n][m], bias, (tile0 + n) * 16 + g * 4, outs), token0 + wave_m * (16 * MW) + m * 16 + r,
                       (tile0 + n) * 16 + g * 4, rows, outs);
  }
}

template <typename TY, bool GATED>
int launch_wide(const void* x, const void* wp, void* y, int rows, int outs, int k, int k_tiles, int n_tiles,
                hipStream_t stream, const float* bias) {
  const int n_blocks = (n_tiles * 16 + kWideN - 1) / kWideN;
  // 256 tokens per block when that still gives every compute unit its two blocks, else 128
  const bool tall = static_cast<long>(n_blocks) * ((rows + 255) / 256) >= 512;
  const int block_tokens = tall ? 256 : 128;
  const int m_blocks = (rows + block_tokens - 1) / block_tokens;
  const long blocks = static_cast<long>((n_blocks + kXcds - 1) / kXcds) * kXcds * m_blocks;
  if (blocks > 0x7fffffffL || static_cast<long>(rows) * k * 2 >= (1L << 32)) return -2;
  if (tall)
    linear_wide_kernel<TY, 8, GATED><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
        static_cast<const bf16_t*>(x), static_cast<const uintx4*>(wp), static_cast<TY*>(y), rows, outs, k, k_tiles,
        n_tiles, n_blocks, m_blocks, GATED ? nullptr : bias);
  else
    linear_wide_kernel<TY, 4, GATED><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
        static_cast<const bf16_t*>(x), static_cast<const uintx4*>(wp), static_cast<TY*>(y), rows, outs, k, k_tiles,
        n_tiles, n_blocks, m_blocks, GATED ? nullptr : bias);
  return AKV_LAUNCH_STATUS();
}

// x [rows, k] row-major -> [tile of 16 rows][k / 8][16 rows][8]: a thread moves 16 bytes; consecutive threads read
// consecutive pieces of a row.  Rows beyond `rows` of the last tile are not written (their lanes never load them).
__global__ void pack_rows_kernel(const uintx4* __restrict__ x, uintx4* __restrict__ xp, int rows, int pieces) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= static_cast<long>(rows) * pieces) return;
  const int row = static_cast<int>(index / pieces), piece = static_cast<int>(index % pieces);
  xp[(static_cast<long>(row / 16) * pieces + piece) * 16 + row % 16] = x[index];
}

}  // namespace

extern "C" int akv_pack_rows(const void* x, void* xp, int rows, int k, hipStream_t stream) {
  if (rows <= 0) return 0;
  if ((k & 7) != 0) return -2;
  const long pieces = static_cast<long>(rows) * (k / 8);
  pack_rows_kernel<<<static_cast<unsigned>((pieces + 255) / 256), 256, 0, stream>>>(
      static_cast<const uintx4*>(x), static_cast<uintx4*>(xp), rows, k / 8);
  return AKV_LAUNCH_STATUS();
}

namespace {
template <bool GATED>
int linear_packed(const void* x, const void* wp, void* y, int y_dtype, int rows, int outs, int k, int n_tiles,
                  int k_tiles, int x_packed, hipStream_t stream, const float* bias = nullptr) {
  if (rows <= 64) {
    if (y_dtype == kF32) return dispatch_skinny<float, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
    if (y_dtype == kBF16) return dispatch_skinny<bf16_t, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, x_packed, stream, bias);
    return -1;
  }
  if (x_packed) return -2;  // only the products of up to 64 rows read packed activations
  if (y_dtype == kF32) return launch_wide<float, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, stream, bias);
  if (y_dtype == kBF16) return launch_wide<bf16_t, GATED>(x, wp, y, rows, outs, k, k_tiles, n_tiles, stream, bias);
  return -1;
}
}  // namespace

// x [rows, k] bfloat16 row-major; wp the packed weight of `n_tiles` x `k_tiles` tiles; y [rows, outs] bfloat16 or
// float32.  k must be a multiple of 8 (a lane's 16-byte read of x must lie inside or outside the row as a whole).
// `x_packed` (rows <= 64 only): x is not row-major but [tile of 16 rows][k / 8][16 rows][8], what akv_pack_rows writes.
// `bias` [outs] float32 or null: added to the float32 sums before they are rounded.
extern "C" int akv_linear_packed(const void* x, const void* wp, void* y, int y_dtype, int rows, int outs, int k,
                                 int n_tiles, int k_tiles, int x_packed, const float* bias, hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if ((k & 7) != 0 || n_tiles * 16 < outs || k_tiles * 32 < k) return -2;
  return linear_packed<false>(x, wp, y, y_dtype, rows, outs, k, n_tiles, k_tiles, x_packed, stream, bias);
}

namespace {
constexpr int kMaxDevices = 64;
void* scratch_of_device[kMaxDevices];   // the array's address on each device, asked for once
std::mutex scratch_guard;

// The address of `scratch` on the current device (every GPU holds its own copy at its own address).
int static_rows(void** address) {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return static_cast<int>(status);
  if (device < 0 || device >= kMaxDevices) return -2;
  std::lock_guard<std::mutex> lock(scratch_guard);
  if (scratch_of_device[device] == nullptr) {
    void* found = nullptr;
    status = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (status != hipSuccess) return static_cast<int>(status);
    if (found == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
    scratch_of_device[device] = found;
  }
  *address = scratch_of_device[device];
  return 0;
}
}  // namespace

// akv_pack_rows followed by akv_linear_packed(x_packed = 1) without any allocation by anybody: the repacked
// activations go to the library's own 4 MiB of static device memory instead of a buffer the caller brings.
// Returns -3 where ceil(rows / 16) * 16 * k bfloat16 do not fit that memory or rows exceed 64.  Nothing needs clearing
// between calls: a call writes every element that it reads (rows beyond `rows` of the last tile are neither).
extern "C" int akv_linear_packed_static(const void* x, const void* wp, void* y, int y_dtype, int rows, int outs, int k,
                                        int n_tiles, int k_tiles, hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if ((k & 7) != 0 || n_tiles * 16 < outs || k_tiles * 32 < k) return -2;
  if (rows > 64 || static_cast<size_t>((rows + 15) / 16 * 16) * k * sizeof(uint16_t) > kStaticRowsBytes) return -3;
  void* packed = nullptr;
  const int found = static_rows(&packed);
  if (found != 0) return found;
  const long pieces = static_cast<long>(rows) * (k / 8);
  pack_rows_kernel<<<static_cast<unsigned>((pieces + 255) / 256), 256, 0, stream>>>(
      static_cast<const uintx4*>(x), static_cast<uintx4*>(packed), rows, k / 8);
  const int status = AKV_LAUNCH_STATUS();
  if (status != 0) return status;
  return linear_packed<false>(packed, wp, y, y_dtype, rows, outs, k, n_tiles, k_tiles, 1, stream);
}

// The gated pair in one pass: wp holds 2 * inter / 16 row tiles, gate tile t at 2t and up tile t at 2t + 1;
// y [rows, inter] = silu(x Wgate^T) * (x Wup^T).  inter must be a multiple of 16.
extern "C" int akv_linear_packed_swiglu(const void* x, const void* wp, void* y, int y_dtype, int rows, int inter,
                                        int k, int n_tiles, int k_tiles, int x_packed, hipStream_t stream) {
  if (rows <= 0 || inter <= 0) return 0;
  if ((k & 7) != 0 || (inter & 15) != 0 || n_tiles * 8 != inter || k_tiles * 32 < k) return -2;
  return linear_packed<true>(x, wp, y, y_dtype, rows, inter, k, n_tiles, k_tiles, x_packed, stream);
}


// The product of a few rows that are not computed yet: rows = norm(stream_in (+ delta)) as akv_add_rmsnorm norms them
// (bfloat16 activations), normed by every block of the product for itself; stream_out [rows, k] receives
// stream_in + delta and must be another buffer than stream_in.  `gated`: akv_linear_packed_swiglu's packing and result.
// At most 4 rows; k a multiple of 8; -2 where the rows do not fit the block's LDS beside its sums.  `bias` [outs] float32
// or null (never with `gated`).
extern "C" int akv_linear_packed_normed(const float* stream_in, const void* delta, const float* norm_weight, float eps,
                                        float* stream_out, const void* wp, void* y, int rows, int outs, int k,
                                        int n_tiles, int k_tiles, int gated, const float* bias, hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if (rows > 4 || (k & 7) != 0 || k_tiles * 32 < k || stream_in == stream_out ||
      (gated ? ((outs & 15) != 0 || n_tiles * 8 != outs) : n_tiles * 16 < outs))
    return -2;
  NormIn norm{stream_in, static_cast<const bf16_t*>(delta), norm_weight, stream_out, eps, 0};
  if (gated) return launch_skinny<1, 2, bf16_t, true, true>(nullptr, wp, y, rows, outs, k, k_tiles, n_tiles, 0, stream, bias, norm);
  if (rows >= 4 && n_tiles >= 384 && n_tiles < 2048)
    return launch_skinny<1, 2, bf16_t, false, true>(nullptr, wp, y, rows, outs, k, k_tiles, n_tiles, 0, stream, bias, norm);
  return launch_skinny<1, 1, bf16_t, false, true>(nullptr, wp, y, rows, outs, k, k_tiles, n_tiles, 0, stream, bias, norm);
}
