// bfloat16 matrix products y = x W^T for some tens to some hundreds of rows (a decode step of many requests, a short
// prompt, a small portion beside decoding requests) on the matrix cores, float32 accumulation.
//
// With so many rows the weights are still read once and memory still sets the pace, but a weight tile of 1 KB now
// meets one activation operand of 1 KB per 16 rows.  If every wave fetched those operands for itself, the caches
// would move several times what memory delivers.  Here the waves of a block share them:
//   * a block owns a band of A * RT row tiles of the packed weight (see gemm_mfma.hip for the packing); 2 A of its
//     waves multiply, A along the band x 2 along k (each half of the block's k);
//   * per stage of S k-tiles the block's activations [16 * MT rows][S * 32 k] of either k half go through LDS,
//     double-buffered, one barrier per stage, as tiles of the matrix-core operand (16 rows x 32 k, 1 KB; the places
//     of a tile's 64 pieces are permuted so that neither readers nor writers meet in a bank).  Four further waves do
//     nothing but fetch them, whole cache lines of a few rows per load,
//     two stages ahead: a wave's loads come back in the order they were issued, so a multiplying wave that fetched
//     activations between its weight loads would have to wait for ALL weights it has asked for before it could use
//     the activations - which brings the weights' distance down to one stage (measured: 1.6 us per stage, whatever
//     the depth of the ring);
//   * every multiplying wave streams its own RT row tiles straight from memory into a ring of G operand register
//     sets, G - 1 stages ahead.  A load takes about two microseconds to come back, so what sets the pace is how much
//     is on its way: a product with few row tiles has few blocks, and each wave of them then keeps 12 KB and more in
//     flight.
// More than 16 * MT rows are taken by several blocks per band; these sit next to each other on one XCD, so that the
// weights they share come from memory once (and are then not marked as read-once).
//
// GATED: the packed matrix alternates gate and up tiles (RT = 2 gives a wave one pair); what is stored is
// silu(gate) * up from the float32 sums.

#include <mutex>
#include <type_traits>

#include "common.h"
#include "mfma_tiles.h"
#include "api.h"

using namespace akv;

namespace {

constexpr int kHalves = 2;   // waves along k (A waves along the band of row tiles: 2, 3 or 4)
constexpr int kFetchers = 4;

// What a product does beyond y = x W^T in a step of many rows that keeps the residual sum and the norm between two
// branches out of kernels of their own (all pointers null: nothing).
//   ADDS (`stream`; never gated, y bfloat16): the branch's last product rounds its result to bfloat16, adds it to the
//   float32 residual sum in place, stores the new sum times the weight of the norm that follows (`gain`) as y, and
//   leaves, per band of its row tiles and row, the sum of squares of the band's new values in `sums_out`.
//   ROWSCALED (`sums_in`): x holds such rows - the residual sum times the norm's weight, not yet divided by the
//   rows' root mean square.  The division commutes with the product: every float32 sum is multiplied by
//   rsqrt(mean of squares + eps) of its row before bias, activation and rounding; the row's sum of squares is added
//   up from the `groups_in` partial sums that the ADDS product left (in the order of the bands, by the fetching waves,
//   who asked for them before the stream began).  Against a norm kernel's rows (scaled, rounded, times the weight,
//   rounded) the operand is rounded once and the scale stays in float32.
struct MidFold {
  float* stream;          // ADDS: [rows, outs]
  const float* gain;      // ADDS: [outs]
  float* sums_out;        // ADDS: [bands][sum_stride]
  const float* sums_in;   // ROWSCALED: [groups_in][sum_stride]
  int groups_in;
  int sum_stride;         // rows of the step, rounded up to a multiple of 16
  float eps, inv_k;       // ROWSCALED: 1 / width of the normed rows (this product's k)
};
constexpr int kMostSums = 40;   // partial sums of a row that one fetching thread adds up (it holds them in registers)
// threads of the fetching waves that share a row's partial sums
template <int MT> constexpr int kSumChunks = (kFetchers * 64) / (MT * 16);
constexpr int kExtraFloats = 256 + 4 * 128;   // LDS behind the staging memory: the rows' sums by chunk; squares by wave

template <int MT> constexpr int kStage = MT <= 4 ? 4 : 2;     // k-tiles per stage and k half

// Where the 16 bytes of operand lane (r, g) lie inside the 1 KB tile of the stage's k-tile u.  A multiplying wave reads a
// tile's 64 places at once, a fetching wave writes, per load, the places of a few rows r and all (u, g): with the
// row's lowest bits turned by (u, g) both spread evenly over the memory's banks.
__device__ __forceinline__ int slot_of(int u, int g, int r) { return g * 16 + (r ^ ((u * 4 + g) & 7)); }

template <int A, int MT, int RT, int G, bool GATED, typename TY>
__global__ __launch_bounds__((A * kHalves + kFetchers) * 64) void linear_mid_kernel(const bf16_t* __restrict__ x, const uintx4* __restrict__ wp,
                                                              TY* __restrict__ y, float* __restrict__ partial,
                                                              unsigned* __restrict__ counters, int rows, int outs, int k,
                                                              int k_tiles, int n_tiles, int bands, int parts,
                                                              int part_tiles, int m_blocks, const float* __restrict__ bias,
                                                              const MidFold fold) {
  constexpr int S = kStage<MT>;
  constexpr int kBlockRows = MT * 16, kChunks = kSumChunks<MT>;
  const bool rowscaled = fold.sums_in != nullptr;
  constexpr int kAlong = A, kMultipliers = A * kHalves;
  constexpr int kTiles = kHalves * S * MT;        // activation tiles of one stage
  constexpr int kLoads = kTiles / kFetchers;      // of which every fetching wave brings this many
  static_assert(kTiles % kFetchers == 0, "the stage's tiles are dealt to the fetching waves");
  static_assert(G % 2 == 0, "a ring position must always meet the same staging buffer");
  extern __shared__ uintx4 staged[];              // [2][kTiles][64]; afterwards the sums of the second k half, then a flag
  float* extra = reinterpret_cast<float*>(staged + 2 * kTiles * 64);   // [kExtraFloats]

  // which work: blocks that share weights (same band and part of k, other rows) are neighbours on one XCD
  const int xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
  const int item = (slot / m_blocks) * kXcds + xcd, m_block = slot % m_blocks;
  if (item >= bands * parts) return;
  const int band = item / parts, part = item % parts;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int row0 = m_block * MT * 16;
  const int kb0 = part * part_tiles, kb1 = min(k_tiles, kb0 + part_tiles);   // the block's k-tiles
  const int per_half = (kb1 - kb0 + kHalves - 1) / kHalves;
  const int stages = (per_half + S - 1) / S;
  const uintx4 zero = {0u, 0u, 0u, 0u};

  if (wave >= kMultipliers) {
    // ---- a fetching wave.  A load brings 1 KB of the stage's activations as they lie in memory: 16 / S rows, of each
    //      the S * 32 consecutive k of one k half (whole cache lines; lane (r, g) of the operand asking for its own
    //      16 bytes would touch 16 rows a load and keep the cache's tag lookup busier than the weights do).  A stage
    //      has kTiles such loads; this wave brings i = f, f + 4, ... of every stage, two stages ahead of the
    //      multiplying waves, and files each 16-byte piece at its place of the operand tile (see `slot_of`).
    const int f = wave - kMultipliers;
    constexpr int kRowsPerLoad = 16 / S;
    const int row_in_load = lane / (4 * S), piece = lane % (4 * S);   // piece = k-tile of the stage * 4 + chunk of 8
    // Every load is issued whatever it asks for - rows beyond the last, k beyond this half's part are asked for at an
    // address that exists - and what must count as zero is zeroed when it is filed: with a test per load the compiler
    // cannot count the loads between a tile and its use and waits for the stage after it as well.
    uintx4 fetched[2][kLoads];
    unsigned there[2];             // bit j: load j of the set brought something that exists
    auto fetch_rows = [&](int stage, uintx4 (&into)[kLoads], unsigned& exists) {
      exists = 0u;
#pragma unroll
      for (int j = 0; j < kLoads; ++j) {
        const int i = f + kFetchers * j;
        const int h = i / (S * MT), group = i % (S * MT);
        const int kt = kb0 + h * per_half + stage * S + piece / 4;
        const int row = row0 + group * kRowsPerLoad + row_in_load, col = kt * 32 + (piece % 4) * 8;
        const bool real = kt < min(kb1, kb0 + (h + 1) * per_half) && row < rows && col < k;
        exists |= real ? 1u << j : 0u;
        into[j] = *reinterpret_cast<const uintx4*>(x + static_cast<size_t>(min(row, rows - 1)) * k + min(col, k - 8));
      }
    };
    auto file_rows = [&](int buffer, const uintx4 (&from)[kLoads], unsigned exists) {
#pragma unroll
      for (int j = 0; j < kLoads; ++j) {
        const int i = f + kFetchers * j;
        const int h = i / (S * MT), group = i % (S * MT);
        const int row = group * kRowsPerLoad + row_in_load;          // of the block's MT * 16
        const int u = piece / 4, g = piece % 4;
        staged[(buffer * kTiles + (h * S + u) * MT + row / 16) * 64 + slot_of(u, g, row % 16)] = (exists >> j & 1u) ? from[j] : zero;
      }
    };
    // ROWSCALED: thread (chunk, row) asks for the partial sums chunk, chunk + kChunks, ... of its row before anything
    // else (loads come back in the order they were asked for: asked for later, they would stand between the first
    // stages' activations and their filing) and adds them up when the stream is over.
    const int ft = threadIdx.x - kMultipliers * 64, sum_row = ft % kBlockRows, sum_chunk = ft / kBlockRows;
    float partials[kMostSums];
    if (rowscaled) {
      const float* from = fold.sums_in + min(row0 + sum_row, fold.sum_stride - 1);
#pragma unroll
      for (int i = 0; i < kMostSums; ++i)
        partials[i] = from[static_cast<size_t>(min(sum_chunk + kChunks * i, fold.groups_in - 1)) * fold.sum_stride];
    }
    fetch_rows(0, fetched[0], there[0]);
    fetch_rows(1, fetched[1], there[1]);
    __builtin_amdgcn_sched_barrier(0);
    int first = 0;
    for (; first + 2 <= stages; first += 2) {       // (pairs of stages, no test inside)
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        // (the fences keep the zeroing of a set's pieces where it is written - behind the other set's loads -: moved
        // up by the compiler it waits for loads that were meant to have a stage's time)
        file_rows(d, fetched[d], there[d]);
        __builtin_amdgcn_sched_barrier(0);
        fetch_rows(first + d + 2, fetched[d], there[d]);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
      }
    }
    if (first < stages) {
      file_rows(0, fetched[0], there[0]);
      __syncthreads();
    }
    if (rowscaled) {
      float total = 0.f;
#pragma unroll
      for (int i = 0; i < kMostSums; ++i)
        if (sum_chunk + kChunks * i < fold.groups_in) total += partials[i];
      if (sum_chunk < kChunks) extra[sum_chunk * kBlockRows + sum_row] = total;
      __syncthreads();   // (the multiplying waves meet it when their stream is over)
    }
    return;
  }

  // ---- a multiplying wave
  const int along = wave % kAlong, half = wave / kAlong;
  const int tile0 = (band * kAlong + along) * RT;
  const int mine0 = kb0 + half * per_half, mine1 = min(kb1, mine0 + per_half);
  const bool shared_weights = m_blocks > 1;       // other blocks read the same tiles: let the caches keep them
  floatx4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // The loads of a stage's weight tiles are the same instructions at every turn, with no test among them: tiles
  // beyond the matrix or beyond this wave's part of k are asked for at the last tile that exists instead - their
  // sums are never stored, or meet activation tiles that the fetching waves have filled with zeros.  (With a test
  // per load the compiler cannot count how many younger loads stand between a tile and its use, and waits for ALL
  // loads - the ones just issued for a later stage included - before it multiplies: the ring was never ahead.)
  auto fetch_weights = [&](int stage, uintx4 (&a)[RT][S], auto once) {
    const int kt = mine0 + stage * S;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int u = 0; u < S; ++u) {
        const uintx4* from = wp + lane + tile_index<GATED>(min(tile0 + rt, n_tiles - 1), min(kt + u, k_tiles - 1), k_tiles) * 64;
        a[rt][u] = decltype(once)::value ? load_once(from) : *from;
      }
  };
  auto multiply = [&](int buffer, const uintx4 (&a)[RT][S]) {
    const uintx4* tiles = staged + (buffer * kTiles + half * S * MT) * 64;
#pragma unroll
    for (int u = 0; u < S; ++u) {
      uintx4 b[MT];
      const int slot = slot_of(u, g, r);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[mt] = tiles[(u * MT + mt) * 64 + slot];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = mfma16(a[rt][u], b[mt], acc[rt][mt]);
    }
  };

  // The turns of the ring: G stages a turn, no test inside a turn; what is left after the last whole turn (fewer than
  // G stages) runs with tests.  Loads for stages beyond the last one bring a tile that exists and nobody multiplies.
  auto stream = [&](auto once) {
    uintx4 a[G][RT][S];
#pragma unroll
    for (int d = 0; d < G - 1; ++d) fetch_weights(d, a[d], once);
    int first = 0;
    for (; first + G <= stages; first += G) {
#pragma unroll
      for (int d = 0; d < G; ++d) {
        __syncthreads();          // the stage's activations are in LDS
        fetch_weights(first + d + G - 1, a[(d + G - 1) % G], once);
        __builtin_amdgcn_sched_barrier(0);   // (left alone the compiler moves these loads behind the products: no ring)
        multiply(d & 1, a[d]);
      }
    }
#pragma unroll
    for (int d = 0; d < G - 1; ++d) {
      if (first + d < stages) {
        __syncthreads();
        fetch_weights(first + d + G - 1, a[(d + G - 1) % G], once);
        __builtin_amdgcn_sched_barrier(0);
        multiply(d & 1, a[d]);
      }
    }
  };
  if (shared_weights) stream(std::false_type{});
  else stream(std::true_type{});

  // the two k halves: the second hands its sums over through LDS, the first adds them to its own
  __syncthreads();
  float* sums = reinterpret_cast<float*>(staged) + static_cast<size_t>(along) * RT * MT * 256;
  if (half == 1) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        *reinterpret_cast<floatx4*>(sums + ((rt * MT + mt) * 64 + lane) * 4) = acc[rt][mt];
  }
  __syncthreads();
  if (half == 0) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const floatx4 other = *reinterpret_cast<const floatx4*>(sums + ((rt * MT + mt) * 64 + lane) * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rt][mt][i] += other[i];
      }
  }
  if (parts > 1) {
    // k is cut over blocks as well: every block leaves its sums in `partial`; the block of a band that arrives last
    // adds the parts in the order of their k ranges (whichever block that is, the bits are the same) and stores.
    const size_t block_floats = static_cast<size_t>(kAlong) * RT * MT * 256;
    float* band_parts = partial + (static_cast<size_t>(m_block) * bands + band) * parts * block_floats;
    // The parts are stored and loaded with device scope themselves - such accesses go through to where all XCDs see
    // them -; the counter's tick is the release and the acquire that orders them (see `arrive` in common.h).
    if (half == 0) {
      float* mine = band_parts + part * block_floats + static_cast<size_t>(along) * RT * MT * 256;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) publish(mine + ((rt * MT + mt) * 4 + i) * 64 + lane, acc[rt][mt][i]);
    }
    __syncthreads();                   // (the fetching waves have gone; all multiplying waves have stored)
    if (threadIdx.x == 0) {
      unsigned* counter = counters + m_block * bands + band;
      const bool last = arrive(counter) == static_cast<unsigned>(parts - 1);
      if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
      *reinterpret_cast<volatile unsigned*>(staged) = last ? 1u : 0u;   // (the sums that lay here have been read)
    }
    __syncthreads();
    if (*reinterpret_cast<volatile unsigned*>(staged) == 0u) return;
    if (half == 0) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
      for (int p = 0; p < parts; ++p) {
        const float* theirs = band_parts + p * block_floats + static_cast<size_t>(along) * RT * MT * 256;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[rt][mt][i] += collect(theirs + ((rt * MT + mt) * 4 + i) * 64 + lane);
      }
    }
  }
  if (half != 0) return;
  if (rowscaled) {   // every sum times its row's 1 / root mean square
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float total = 0.f;
#pragma unroll
      for (int c = 0; c < kChunks; ++c) total += extra[c * kBlockRows + mt * 16 + r];
      const float scale = rsqrtf(total * fold.inv_k + fold.eps);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rt][mt][i] *= scale;
    }
  }
  constexpr bool kMayAdd = !GATED && std::is_same<TY, bf16_t>::value;
  if constexpr (kMayAdd) {
    if (fold.stream != nullptr) {
      // What the sums are added to - the residual sum's values at this wave's outputs, and the norm's weight there -
      // is asked for in one go, every load whatever its place (places beyond the matrix or the rows ask at one that
      // exists and are not used): loads behind tests would be waited for one by one, a trip to memory each.  (Asked
      // for before the exchanges of sums, which would hide their way, they take the registers that the exchange
      // needs to have its own loads in flight together: 24 -> 83 us at 128 rows.)
      const bool whole_quads = (outs & 3) == 0;
      float4 held[RT][MT], weight_held[RT];
      if (whole_quads) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          const int feature = max(0, min((tile0 + rt) * 16 + g * 4, outs - 4));
          weight_held[rt] = *reinterpret_cast<const float4*>(fold.gain + feature);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            held[rt][mt] = *reinterpret_cast<const float4*>(fold.stream + static_cast<size_t>(min(row0 + mt * 16 + r, rows - 1)) * outs + feature);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      float squares[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        squares[mt] = 0.f;
        const int row = row0 + mt * 16 + r;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          const int feature = (tile0 + rt) * 16 + g * 4;
          if (tile0 + rt >= n_tiles || row >= rows || feature >= outs) continue;
          const floatx4 product = plus_bias(acc[rt][mt], bias, feature, outs);
          float* sum_at = fold.stream + static_cast<size_t>(row) * outs + feature;
          if (whole_quads) {     // (then feature + 3 < outs: the features of a quad exist together)
            const float4 before = held[rt][mt], weight = weight_held[rt];
            floatx4 now = {before.x + rounded<bf16_t>(product[0]), before.y + rounded<bf16_t>(product[1]),
                           before.z + rounded<bf16_t>(product[2]), before.w + rounded<bf16_t>(product[3])};
            *reinterpret_cast<float4*>(sum_at) = make_float4(now[0], now[1], now[2], now[3]);
            squares[mt] += now[0] * now[0] + now[1] * now[1] + now[2] * now[2] + now[3] * now[3];
            store4<bf16_t>(y + static_cast<size_t>(row) * outs + feature,
                           floatx4{now[0] * weight.x, now[1] * weight.y, now[2] * weight.z, now[3] * weight.w});
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (feature + i < outs) {
                const float now = sum_at[i] + rounded<bf16_t>(product[i]);
                sum_at[i] = now;
                squares[mt] += now * now;
                y[static_cast<size_t>(row) * outs + feature + i] = from_float<bf16_t>(now * fold.gain[feature + i]);
              }
          }
        }
        squares[mt] += __shfl_xor(squares[mt], 16, kWave);
        squares[mt] += __shfl_xor(squares[mt], 32, kWave);
      }
      // the band's sum per row: the waves along the band, added in their order
      float* by_wave = extra + 256;
      if (g == 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) by_wave[along * kBlockRows + mt * 16 + r] = squares[mt];
      }
      __syncthreads();   // (only the first k half's waves are left)
      for (int row = along * 64 + lane; row < kBlockRows; row += kAlong * 64) {
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < kAlong; ++w) total += by_wave[w * kBlockRows + row];
        if (row0 + row < fold.sum_stride) fold.sums_out[static_cast<size_t>(band) * fold.sum_stride + row0 + row] = total;
      }
      return;
    }
  }
  if constexpr (GATED) {
    static_assert(RT % 2 == 0, "a wave must own gate and up tiles in pairs");
#pragma unroll
    for (int rt = 0; rt < RT; rt += 2)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        if (tile0 + rt < n_tiles)
          store_tile<TY>(y, silu_times(acc[rt][mt], acc[rt + 1][mt]), row0 + mt * 16 + r, ((tile0 + rt) >> 1) * 16 + g * 4,
                         rows, outs);
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        if (tile0 + rt < n_tiles)
          store_tile<TY>(y, plus_bias(acc[rt][mt], bias, (tile0 + rt) * 16 + g * 4, outs), row0 + mt * 16 + r,
                         (tile0 + rt) * 16 + g * 4, rows, outs);
  }
}

struct MidPlan {
  int along, mt, rt, depth, bands, parts, part_tiles, m_blocks;
  size_t partial_floats, counters;
};

constexpr size_t kMostPartialFloats = 8u << 20;   // 32 MB: more than that is not worth a cut of k over blocks

// How a product of `rows` rows is cut into blocks.  A compute unit draws little more than 20 GB/s from memory however
// much its waves ask for, so a product streams at the device's rate only when every compute unit has a block, and
// the blocks are equal: the cut (waves along the band, row tiles per wave, blocks along k) that keeps the busiest
// compute unit's share smallest is taken, counted in weight tiles (measured at Qwen3-8B shapes: the best cut of every
// product was one that gives each of the 256 compute units exactly one block).  `along`, `rt`, `depth` and `parts`
// of 0 leave the choice to the sizes; others force it (for measurements).
MidPlan plan_mid(int rows, int n_tiles, int k_tiles, bool gated, int along, int rt, int depth, int parts) {
  MidPlan best{};
  double best_cost = -1.0;
  const int kComputeUnits = device_facts().compute_units;
  // tiles of 16 rows: up to eight a block, dealt evenly to the blocks (132 rows are two blocks of five tiles, not
  // one of eight and one that multiplies zeros)
  const int row_tiles = (rows + 15) / 16;
  const int m_blocks = (row_tiles + 7) / 8;
  const int mt = row_tiles < 2 ? 2 : (row_tiles + m_blocks - 1) / m_blocks;
  for (int a = 2; a <= 4; ++a) {
    if (along != 0 && a != along) continue;
    for (int r = 1; r <= 2; ++r) {
      if ((gated && r != 2) || (rt != 0 && r != rt)) continue;
      for (int cut = 1; cut <= 16; cut *= 2) {
        if (parts != 0 && cut != parts) continue;
        if (parts == 0 && cut > 1 && k_tiles / cut < 2 * kHalves * 4) break;   // a block keeps a few stages of work
        MidPlan p{};
        p.along = a, p.mt = mt, p.rt = r, p.m_blocks = m_blocks;
        p.bands = (n_tiles + a * r - 1) / (a * r);
        p.part_tiles = (k_tiles + cut - 1) / cut;
        p.parts = (k_tiles + p.part_tiles - 1) / p.part_tiles;
        p.partial_floats = p.parts > 1 ? static_cast<size_t>(m_blocks) * p.bands * p.parts * a * r * mt * 256 : 0;
        p.counters = p.parts > 1 ? static_cast<size_t>(m_blocks) * p.bands : 0;
        if (parts == 0 && p.partial_floats > kMostPartialFloats) continue;
        const long blocks = static_cast<long>(p.bands) * p.parts * m_blocks;
        const long rounds = (blocks + kComputeUnits - 1) / kComputeUnits;
        // What the busiest compute unit moves, counted in weight tiles (1 KB from memory, about 50 ns at the rate a
        // unit gets when all read): its blocks' weight tiles; the activation tiles they stage through LDS, which come
        // from the caches and cost two thirds of a weight tile each (fitted: the down product of 4,096 x 12,288 at 64
        // rows takes 45.7 us with 768 activation tiles a block, 33.2 with 384); what a block costs before and after
        // its stream, about 1.2 us (the down product of 5,120 x 17,408 at 32 rows: 57 us as 1,280 blocks of 34 k tiles,
        // 42 us as 216 blocks of 136); and the exchange of partial sums (fitted on the first product: 9 us for 8 parts
        // of 8 row tiles x 4 tiles of rows).  Of equal cuts the one with two row tiles per wave wins, then the one
        // with more waves along the band, then the one with fewer parts.  (Over 40 products of Qwen3-8B and -14B
        // shapes at 24 to 256 rows the cut chosen so takes 1.3 % longer than the best of all cuts, on average.)
        double cost = static_cast<double>(rounds) * (static_cast<double>(a) * r * p.part_tiles + 0.68 * mt * p.part_tiles + 24.0);
        if (p.parts > 1) cost += static_cast<double>(a) * r * mt * p.parts / 1.6;
        if (a == 2) cost *= 0.96;   // (blocks of eight waves: two share a compute unit, one's loads fill the other's waits)
        cost += 0.05 * (2 - r) + 0.01 * (4 - a) + 0.001 * p.parts;
        if (best_cost < 0.0 || cost < best_cost) best = p, best_cost = cost;
      }
    }
  }
  // two row tiles a wave: a ring of two register sets (a deeper one does not fit the registers); one row tile: of four
  // (measured: never slower than two).  `depth` can only ask for what the row tiles allow.
  if (depth != 0 && depth != (best.rt == 2 ? 2 : 4)) return MidPlan{};
  best.depth = best.rt == 2 ? 2 : 4;
  return best;
}

template <int A, int MT, int RT, int G, bool GATED, typename TY>
int launch_mid(const MidPlan& p, const void* x, const void* wp, void* y, float* partial, unsigned* counters, int rows,
               int outs, int k, int k_tiles, int n_tiles, const float* bias, const MidFold& fold, hipStream_t stream) {
  constexpr size_t staging = 2 * kHalves * kStage<MT> * MT * 1024;
  static_assert(staging >= static_cast<size_t>(A) * RT * MT * 1024, "the sums of a k half must fit the staging memory");
  static_assert(staging <= 64 * 1024, "the staging memory of a block");
  static_assert(kSumChunks<MT> * MT * 16 <= 256 && A * MT * 16 <= 4 * 128, "what lies behind the staging memory");
  constexpr size_t lds = staging + kExtraFloats * 4;
  if (fold.sums_in != nullptr && fold.groups_in > kSumChunks<MT> * kMostSums) return -2;
  if (lds > 64 * 1024) {   // more than a block may have without asking: asked once per kernel and device
    static std::mutex guard;
    static bool asked[64] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return -2;
    std::lock_guard<std::mutex> lock(guard);
    if (!asked[device]) {
      const hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_mid_kernel<A, MT, RT, G, GATED, TY>),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (status != hipSuccess) return static_cast<int>(status);
      asked[device] = true;
    }
  }
  const long items = static_cast<long>(p.bands) * p.parts;
  const long blocks = (items + kXcds - 1) / kXcds * kXcds * p.m_blocks;
  if (blocks > 0x7fffffffL) return -2;
  linear_mid_kernel<A, MT, RT, G, GATED, TY><<<static_cast<unsigned>(blocks), (A * kHalves + kFetchers) * 64, lds, stream>>>(
      static_cast<const bf16_t*>(x), static_cast<const uintx4*>(wp), static_cast<TY*>(y), partial, counters, rows, outs,
      k, k_tiles, n_tiles, p.bands, p.parts, p.part_tiles, p.m_blocks, GATED ? nullptr : bias, fold);
  return AKV_LAUNCH_STATUS();
}

template <bool GATED, typename TY>
int dispatch_mid(const MidPlan& p, const void* x, const void* wp, void* y, float* partial, unsigned* counters, int rows,
                 int outs, int k, int k_tiles, int n_tiles, const float* bias, const MidFold& fold, hipStream_t stream) {
#define AKV_MID(A_, MT_, RT_, G_) \
  if (p.along == A_ && p.mt == MT_ && p.rt == RT_ && p.depth == G_) \
    return launch_mid<A_, MT_, RT_, G_, GATED, TY>(p, x, wp, y, partial, counters, rows, outs, k, k_tiles, n_tiles, bias, fold, stream)
#define AKV_MID_ROWS(A_, RT_, G_) \
  AKV_MID(A_, 2, RT_, G_); AKV_MID(A_, 3, RT_, G_); AKV_MID(A_, 4, RT_, G_); AKV_MID(A_, 5, RT_, G_); \
  AKV_MID(A_, 6, RT_, G_); AKV_MID(A_, 7, RT_, G_); AKV_MID(A_, 8, RT_, G_)
#define AKV_MID_ALONG(RT_, G_) AKV_MID_ROWS(2, RT_, G_); AKV_MID_ROWS(3, RT_, G_); AKV_MID_ROWS(4, RT_, G_)
  AKV_MID_ALONG(2, 2);
  if constexpr (!GATED) {
    AKV_MID_ALONG(1, 4);
  }
#undef AKV_MID_ALONG
#undef AKV_MID_ROWS
#undef AKV_MID
  return -2;
}

}  // namespace

// What akv_linear_mid needs beside its operands for this product: floats of `partial` and unsigned integers of
// `counters` (both 0 where k is not cut over blocks).  `counters` must be zero before the first launch that uses it;
// every launch leaves it zero again.  Launches that may run at the same time must not share the two.
extern "C" int akv_linear_mid_workspace(int rows, int n_tiles, int k_tiles, int gated, int along, int rt, int depth,
                                        int parts, long* partial_floats, long* counters) {
  const MidPlan p = plan_mid(rows, n_tiles, k_tiles, gated != 0, along, rt, depth, parts);
  *partial_floats = static_cast<long>(p.partial_floats);
  *counters = static_cast<long>(p.counters);
  return 0;
}

// x [rows, k] bfloat16 row-major, 1 <= rows; wp the packed weight; y [rows, outs] (gated: [rows, inter], wp as for
// akv_linear_packed_swiglu).  `along` (waves along a band: 2..4), `rt` (row tiles per wave, 1 or 2), `depth`
// (register sets of the weight ring: 2 with rt = 2, 4 with rt = 1) and `parts` (blocks along k, a power of two) may be 0: chosen here.
// `partial_floats` and `counter_words` say how much `partial` and `counters` hold: a cut that needs more
// (akv_linear_mid_workspace tells) is refused with -3 and nothing is launched.  `bias` [outs] float32 or null (never with
// `gated`): added to the float32 sums before they are rounded.
namespace {
int linear_mid(const void* x, const void* wp, void* y, int y_dtype, float* partial, long partial_floats,
               unsigned* counters, long counter_words, int rows, int outs, int k, int n_tiles, int k_tiles, int gated,
               int along, int rt, int depth, int parts, const float* bias, const MidFold& fold, hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if ((k & 7) != 0 || k_tiles * 32 < k) return -2;
  if (gated ? ((outs & 15) != 0 || n_tiles * 8 != outs) : n_tiles * 16 < outs) return -2;
  if (gated && bias != nullptr) return -2;
  if (along < 0 || along == 1 || along > 4 || rt < 0 || rt > 2 || depth < 0 || parts < 0 || (parts & (parts - 1)) != 0) return -2;
  const MidPlan p = plan_mid(rows, n_tiles, k_tiles, gated != 0, along, rt, depth, parts);
  if (p.along == 0) return -2;
  if (p.parts > 1 && (partial == nullptr || counters == nullptr)) return -2;
  if (p.parts > 1 && (static_cast<long>(p.partial_floats) > partial_floats || static_cast<long>(p.counters) > counter_words)) return -3;
  if (gated) {
    if (y_dtype == kF32) return dispatch_mid<true, float>(p, x, wp, y, partial, counters, rows, outs, k, k_tiles, n_tiles, bias, fold, stream);
    if (y_dtype == kBF16) return dispatch_mid<true, bf16_t>(p, x, wp, y, partial, counters, rows, outs, k, k_tiles, n_tiles, bias, fold, stream);
    return -1;
  }
  if (y_dtype == kF32) return dispatch_mid<false, float>(p, x, wp, y, partial, counters, rows, outs, k, k_tiles, n_tiles, bias, fold, stream);
  if (y_dtype == kBF16) return dispatch_mid<false, bf16_t>(p, x, wp, y, partial, counters, rows, outs, k, k_tiles, n_tiles, bias, fold, stream);
  return -1;
}
}  // namespace

extern "C" int akv_linear_mid(const void* x, const void* wp, void* y, int y_dtype, float* partial, long partial_floats,
                              unsigned* counters, long counter_words, int rows, int outs, int k, int n_tiles,
                              int k_tiles, int gated, int along, int rt, int depth, int parts, const float* bias,
                              hipStream_t stream) {
  return linear_mid(x, wp, y, y_dtype, partial, partial_floats, counters, counter_words, rows, outs, k, n_tiles, k_tiles,
                    gated, along, rt, depth, parts, bias, MidFold{}, stream);
}

// The bands of row tiles into which akv_linear_mid_adds cuts this product (one partial sum of squares per band and
// row), and the most partial sums per row that akv_linear_mid_rowscaled adds up for a step of `rows` rows.
extern "C" int akv_linear_mid_bands(int rows, int n_tiles, int k_tiles) {
  return plan_mid(rows, n_tiles, k_tiles, false, 0, 0, 0, 0).bands;
}
extern "C" int akv_linear_mid_most_groups(int rows) {
  const int row_tiles = (rows + 15) / 16, m_blocks = (row_tiles + 7) / 8;
  const int mt = row_tiles < 2 ? 2 : (row_tiles + m_blocks - 1) / m_blocks;
  return (kFetchers * 64) / (mt * 16) * kMostSums;
}

// A branch's last product in a step of many rows (see `MidFold`): stream_sum [rows, outs] float32 += bfloat16(x W^T (+
// bias)) in place; y [rows, outs] bfloat16 receives the new sum times `gain` [outs]; sums_out [bands][sum_stride]
// float32 the bands' sums of squares per row (bands: akv_linear_mid_bands; sum_stride >= rows, a multiple of 16).
extern "C" int akv_linear_mid_adds(const void* x, const void* wp, void* y, float* partial, long partial_floats,
                                   unsigned* counters, long counter_words, int rows, int outs, int k, int n_tiles,
                                   int k_tiles, const float* bias, float* stream_sum, const float* gain, float* sums_out,
                                   int sum_stride, hipStream_t stream) {
  if (stream_sum == nullptr || gain == nullptr || sums_out == nullptr || sum_stride < rows || (sum_stride & 15) != 0) return -2;
  MidFold fold{};
  fold.stream = stream_sum, fold.gain = gain, fold.sums_out = sums_out, fold.sum_stride = sum_stride;
  return linear_mid(x, wp, y, kBF16, partial, partial_floats, counters, counter_words, rows, outs, k, n_tiles, k_tiles, 0,
                    0, 0, 0, 0, bias, fold, stream);
}

// The product that reads rows left by akv_linear_mid_adds: y = (x W^T) * rsqrt(sum of squares of the row / k + eps) (+
// bias; gated: silu of the scaled gate times the scaled up), the row's sum added up from sums_in [groups][sum_stride].
// Refused with -2 where `groups` exceeds akv_linear_mid_most_groups(rows).
extern "C" int akv_linear_mid_rowscaled(const void* x, const void* wp, void* y, int y_dtype, float* partial,
                                        long partial_floats, unsigned* counters, long counter_words, int rows, int outs,
                                        int k, int n_tiles, int k_tiles, int gated, const float* bias,
                                        const float* sums_in, int groups, int sum_stride, float eps, hipStream_t stream) {
  if (sums_in == nullptr || groups <= 0 || sum_stride < rows) return -2;
  MidFold fold{};
  fold.sums_in = sums_in, fold.groups_in = groups, fold.sum_stride = sum_stride, fold.eps = eps;
  fold.inv_k = 1.f / static_cast<float>(k);
  return linear_mid(x, wp, y, y_dtype, partial, partial_floats, counters, counter_words, rows, outs, k, n_tiles, k_tiles,
                    gated, 0, 0, 0, 0, bias, fold, stream);
}
