// bfloat16 products of up to 16 rows (decode steps) that take the residual sum and the norm between two products
// into the products themselves, so that a layer of a decode step launches no kernel for either:
//
//   ADDS    a branch's last product (o, down) does not store its result: it rounds it to bfloat16, adds it to the
//           float32 residual sum in place, and leaves the sums of squares of the new residual rows, one partial sum per
//           (row tile of 16 outputs, row) - every output is owned by one lane, so no value depends on an order;
//   SCALED  the product that reads the norm of the residual sum (q/k/v, gate and up) does not read normed rows: every
//           block norms the rows for itself into LDS while its first weights are on their way.  The rows' sums of
//           squares are not formed again: the block's waves add the partial sums in a fixed order and form
//           rsqrt(mean + eps); then every thread norms pieces of 8 values as the norm kernel does - scaled, rounded,
//           times the weight, rounded - and puts them where the matrix cores' operand wants them.
//
//   ROWSCALED  the same reader another way round: the adding product has also left the new rows times the norm's
//           weight as bfloat16 (`rows_out`), and since the division by a row's root mean square commutes with the
//           product, this one multiplies those rows as they are and scales its float32 sums by rsqrt(mean + eps) of
//           their row - the blocks read 2 bytes a value instead of 4 and the weight, and norm nothing (q/k/v at 8
//           rows 19.4 -> 17.5 us, gate and up 40.0 -> 36.7 on cold weights).  Against SCALED an operand is rounded
//           once instead of twice and the scale stays in float32: the same up to roundings, not the same bits.
//
// Otherwise this is the skinny kernel of gemm_mfma.hip for one tile of rows: a wave owns RT row tiles of the packed
// weight and a part of k, streams its tiles once (two groups of registers in turn, loads marked as read-once), the
// parts of k are summed through LDS in a fixed order.  GATED as there (a pair of gate and up tiles, RT = 2).
// The work is numbered in units - (RT row tiles, part of k) - and a block takes as many consecutive units as gives
// every compute unit the same share (plan_decode); where that leaves a row tile's parts in two neighbouring blocks,
// the later of the two finishes the tile from sums that both leave in memory.
// The results equal those of the separate kernels up to the order in which a row's squares, and the parts of k, are
// added.

#include <mutex>

#include "common.h"
#include "mfma_tiles.h"
#include "api.h"

using namespace akv;

namespace {

struct DecodeArgs {
  const bf16_t* x;          // not SCALED: [rows, k] (ROWSCALED: the residual rows times the norm's weight)
  const float* stream;      // SCALED: [rows, k], the residual sum
  const float* sums;        // SCALED, ROWSCALED: [sum_tiles][16] partial sums of squares of the residual rows
  const float* gain;        // SCALED: [k], the norm's weight
  const uintx4* wp;         // the packed weight
  bf16_t* y;                // not ADDS: [rows, outs]
  float* stream_out;        // ADDS: [rows, outs], updated in place
  float* sums_out;          // ADDS: [n_tiles][16]
  bf16_t* rows_out;         // ADDS: [rows, outs] or null: the new residual sum times `gain_out`, for a ROWSCALED reader
  const float* gain_out;    // ADDS: [outs], the weight of the norm that follows (with rows_out)
  const float* bias;        // [outs] or null: added to the sums over k before anything else is done with them (never GATED)
  float eps;
  int sum_tiles, rows, outs, k, k_tiles, n_tiles, k_split, red_floats;
  float* pieces;            // [wave-row][2][RT][4][64]: the sums of a wave-row whose parts of k lie in two blocks
  unsigned int* arrivals;   // [wave-row], zero between launches: how many of the two have left their sums
};

constexpr int kGroup = 4;   // k-tiles per group of loads; two groups are in flight

template <int RT, bool GATED, bool SCALED, bool ADDS, bool ROWSCALED = false>
__global__ __launch_bounds__(768) void linear_decode_kernel(const DecodeArgs a) {
  static_assert(!(GATED && ADDS) && (!GATED || RT == 2), "the gated pair is a wave's two row tiles");
  static_assert(!(ROWSCALED && (SCALED || ADDS)), "a product scales its sums, or norms its rows, or adds itself");
  constexpr int U = kGroup;
  extern __shared__ float red[];   // [wave][RT][4][64] for the sum over the parts of k - SCALED: before that, the rows' scales and the normed rows
  const int lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  // The product's work is cut into units - (wave-row of RT row tiles, part of k) - numbered wave-row by wave-row; a
  // block's waves take consecutive units, whole wave-rows or not.
  const int first_unit = blockIdx.x * waves, unit = first_unit + wave;
  const int wave_row = unit / a.k_split, part = unit % a.k_split;
  const int row_tile = wave_row * RT;
  const int per_part = (a.k_tiles + a.k_split - 1) / a.k_split;
  const int kt0 = part * per_part, kt1 = min(a.k_tiles, kt0 + per_part);
  const bool works = row_tile < a.n_tiles && kt0 < kt1;
  const bool ragged = (a.k & 31) != 0;
  const uintx4 zero = {0u, 0u, 0u, 0u};
  floatx4 acc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Weights: every load is issued whatever the sizes are - a tile beyond the wave's part or the matrix reads the last
  // valid one again and is not used - so that the loop's loads sit behind no branch and the compiler can wait for
  // exactly the group it needs while the next is in flight.
  const int last_tile = max(kt1 - 1, 0);
  const uintx4* w_lane = a.wp + lane;
  uintx4 w0[RT][U], w1[RT][U];
  auto fetch_weights = [&](int kt, uintx4 (&w)[RT][U]) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        w[rt][u] = load_once(w_lane + tile_index<GATED>(min(row_tile + rt, a.n_tiles - 1), min(kt + u, last_tile), a.k_tiles) * 64);
  };
  // SCALED: the rows as the operand wants them, [k tile][k chunk of 8][row] x 16 bytes: lane (r, g) reads chunk g, row r
  constexpr int kScaleFloats = 12 * 16 + 16;   // SCALED: every wave's share of the rows' sums of squares, then the scales
  uintx4* rows_lds = reinterpret_cast<uintx4*>(red + (SCALED ? kScaleFloats : 0));
  fetch_weights(kt0, w0);       // two groups on their way while the rows are normed
  fetch_weights(kt0 + U, w1);
  // ADDS: what the sums will be added to, and the next norm's weight there, are asked for now - in the epilogue they
  // would cost the block's last wave a trip to memory.  (Every output has one owner: nobody changes them meanwhile.)
  float4 held[ADDS ? RT : 1], gain_held[ADDS ? RT : 1];
  const bool quads = (a.outs & 3) == 0;
  if constexpr (ADDS) {
    if (quads) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int feature = max(0, min((min(row_tile + rt, a.n_tiles - 1)) * 16 + g * 4, a.outs - 4));
        held[rt] = *reinterpret_cast<const float4*>(a.stream_out + static_cast<size_t>(min(r, a.rows - 1)) * a.outs + feature);
        gain_held[rt] = *reinterpret_cast<const float4*>((a.gain_out != nullptr ? a.gain_out : a.stream_out) + feature);
      }
    }
  }
  float my_scale = 1.f;         // ROWSCALED: 1 / rms of this lane's row
  if constexpr (SCALED || ROWSCALED) {
    // (Asking for what the norm needs BEFORE the first weights - a wave's loads come back in the order in which they
    // were asked for - was measured and is no gain: 15.0 -> 16.0 us at one row, 23.1 -> 22.8 at eight, q/k/v.)
    // The rows' sums of squares: sum_tiles x 16 partial sums.  The waves share the tiles; a lane adds up quads of
    // rows (lane % 4 fixes which four), the lanes of a wave are folded in a fixed order, then the waves' shares - the
    // same order in every block.
    float* shares = red;
    float* scales = red + 12 * 16;
    {
      const int quads = a.sum_tiles * 4, per_wave = ((quads + waves - 1) / waves + 63) / 64 * 64;
      const int q0 = wave * per_wave, q1 = min(quads, q0 + per_wave);
      float4 part = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
      for (int q = q0 + lane; q < q1; q += 64) {
        const float4 v = reinterpret_cast<const float4*>(a.sums)[q];
        part.x += v.x, part.y += v.y, part.z += v.z, part.w += v.w;
      }
#pragma unroll
      for (int step = 4; step < 64; step <<= 1) {
        part.x += __shfl_xor(part.x, step, kWave);
        part.y += __shfl_xor(part.y, step, kWave);
        part.z += __shfl_xor(part.z, step, kWave);
        part.w += __shfl_xor(part.w, step, kWave);
      }
      if (lane < 4) *reinterpret_cast<float4*>(shares + wave * 16 + lane * 4) = part;
    }
    __syncthreads();
    if (threadIdx.x < 16) {
      float total = 0.f;
      for (int w = 0; w < waves; ++w) total += shares[w * 16 + threadIdx.x];
      scales[threadIdx.x] = static_cast<int>(threadIdx.x) < a.rows ? rsqrtf(total / static_cast<float>(a.k) + a.eps) : 0.f;
    }
    __syncthreads();
    if constexpr (ROWSCALED) my_scale = scales[r];
  }
  if constexpr (SCALED) {
    float* scales = red + 12 * 16;
    auto normed = [&](float4 lo, float4 hi, float4 g0, float4 g1, float scale) {
      const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      const float gains[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      uintx4 packed;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        packed[j] = bf16_pair(rounded<bf16_t>(v[2 * j] * scale) * gains[2 * j], rounded<bf16_t>(v[2 * j + 1] * scale) * gains[2 * j + 1]);
      return packed;
    };
    // A thread takes a column of 8 values and walks down the rows, four rows' loads in flight together (one after
    // the other, every row would cost a trip to the caches); the norm's weights of the column are fetched once.
    constexpr int kRowsTogether = 4;
    const int pieces_per_row = a.k >> 3;
    for (int piece = threadIdx.x; piece < pieces_per_row; piece += blockDim.x) {
      const float4 g0 = *reinterpret_cast<const float4*>(a.gain + piece * 8), g1 = *reinterpret_cast<const float4*>(a.gain + piece * 8 + 4);
      for (int row0 = 0; row0 < a.rows; row0 += kRowsTogether) {
        float4 lo[kRowsTogether], hi[kRowsTogether];
#pragma unroll
        for (int j = 0; j < kRowsTogether; ++j) {
          lo[j] = hi[j] = make_float4(0.f, 0.f, 0.f, 0.f);
          if (row0 + j < a.rows) {
            const float* from = a.stream + static_cast<size_t>(row0 + j) * a.k + piece * 8;
            lo[j] = *reinterpret_cast<const float4*>(from), hi[j] = *reinterpret_cast<const float4*>(from + 4);
          }
        }
#pragma unroll
        for (int j = 0; j < kRowsTogether; ++j)   // piece = k tile * 4 + chunk
          if (row0 + j < a.rows) rows_lds[piece * a.rows + row0 + j] = normed(lo[j], hi[j], g0, g1, scales[row0 + j]);
      }
    }
    __syncthreads();
  }

  // the operand of the rows: lane (r, g) brings row r, 8 values at k = g * 8 of the k-tile.  Rows beyond `rows` read
  // the last row again (their results are never stored); the chunks of a ragged last k-tile beyond k count as zero.
  const int row_read = min(r, a.rows - 1);
  const bool lane_outside = ragged && (a.k_tiles - 1) * 32 + g * 8 >= a.k;
  uintx4 x0[U], x1[U];
  auto fetch_rows = [&](int kt, uintx4 (&x)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int tile = min(kt + u, last_tile);
      const int chunk = (lane_outside && tile == a.k_tiles - 1) ? 0 : g;
      if constexpr (SCALED) x[u] = rows_lds[(tile * 4 + chunk) * a.rows + row_read];
      else x[u] = *reinterpret_cast<const uintx4*>(a.x + static_cast<size_t>(row_read) * a.k + tile * 32 + chunk * 8);
    }
  };
  auto multiply = [&](int kt, const uintx4 (&w)[RT][U], const uintx4 (&x)[U]) {
    if (kt + U <= kt1 && !(ragged && kt + U == a.k_tiles)) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt] = mfma16(w[rt][u], x[u], acc[rt]);
    } else {   // the group at the end of the part: tiles beyond it are left out, the ragged last one loses its lanes
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (kt + u < kt1) {
          const bool drop = lane_outside && kt + u == a.k_tiles - 1;
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) acc[rt] = mfma16(w[rt][u], drop ? zero : x[u], acc[rt]);
        }
    }
  };
  if (works) {
    fetch_rows(kt0, x0);
    fetch_rows(kt0 + U, x1);
    int kt = kt0;
    for (; kt + 2 * U < kt1; kt += 2 * U) {   // two groups are in flight; the one after them holds tiles of the part
      multiply(kt, w0, x0);
      fetch_weights(kt + 2 * U, w0);
      fetch_rows(kt + 2 * U, x0);
      __builtin_amdgcn_sched_barrier(0);      // (the loads stay where they are written: ahead of the other group's products)
      multiply(kt + U, w1, x1);
      fetch_weights(kt + 3 * U, w1);          // (beyond the part: the last tile again, never multiplied - no test, so
      fetch_rows(kt + 3 * U, x1);             //  that the waits above can count the loads behind them)
      __builtin_amdgcn_sched_barrier(0);
    }
    multiply(kt, w0, x0);
    if (kt + U < kt1) multiply(kt + U, w1, x1);
  }

  if (a.k_split > 1) {
    // The parts of k are added up in their order.  The units of this wave's wave-row that the block holds are
    // [lo, hi): every wave leaves its sums in LDS, the wave of unit lo adds them up.  Where the block holds the whole
    // wave-row that is the result.  Otherwise the wave-row's other parts lie in the neighbouring block (never in
    // more than two: a block has at least k_split waves): both leave their sums in `pieces` with device-scope
    // stores and tick `arrivals` (a release and an acquire, see `arrive`); the second to arrive adds piece 0 +
    // piece 1 (the same bits whichever it is), sets the counter back and goes on to the store.  Nobody waits for
    // anybody.
    constexpr int kSet = RT * 4 * 64;
    if constexpr (SCALED || ROWSCALED) __syncthreads();   // the rows (the scales) have been read: their memory takes the sums
    const int row_first = wave_row * a.k_split;
    const int lo = max(first_unit, row_first), hi = min(first_unit + waves, row_first + a.k_split);
    float* mine = red + static_cast<size_t>(wave) * kSet;
    if (unit != lo) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) mine[(rt * 4 + i) * 64 + lane] = acc[rt][i];
    }
    __syncthreads();
    if (unit != lo) return;
    for (int other = 1; other < hi - lo; ++other) {
      const float* theirs = mine + static_cast<size_t>(other) * kSet;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rt][i] += theirs[(rt * 4 + i) * 64 + lane];
    }
    if (hi - lo < a.k_split && row_tile < a.n_tiles) {
      const int piece = lo == row_first ? 0 : 1;
      float* ours = a.pieces + (static_cast<size_t>(wave_row) * 2 + piece) * kSet;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) publish(ours + (rt * 4 + i) * 64 + lane, acc[rt][i]);
      // the wave ticks as one: its lanes' stores precede the one read-modify-write, its lanes' loads follow it
      unsigned int before = 0;
      if (lane == 0) before = arrive(a.arrivals + wave_row);
      before = __shfl(before, 0, kWave);
      if (before == 0u) return;        // the other block will finish this wave-row
      if (lane == 0) __hip_atomic_store(a.arrivals + wave_row, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
      const float* theirs = a.pieces + (static_cast<size_t>(wave_row) * 2 + (1 - piece)) * kSet;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float other = collect(theirs + (rt * 4 + i) * 64 + lane);
          acc[rt][i] = piece == 0 ? acc[rt][i] + other : other + acc[rt][i];
        }
    }
  }
  if (row_tile >= a.n_tiles) return;
  if constexpr (ROWSCALED) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[rt][i] *= my_scale;
  }
  if constexpr (!GATED) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[rt] = plus_bias(acc[rt], a.bias, (row_tile + rt) * 16 + g * 4, a.outs);
  }
  if constexpr (ADDS) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int tile = row_tile + rt;
      if (tile >= a.n_tiles) break;
      const int feature = tile * 16 + g * 4;
      float squares = 0.f;
      if (r < a.rows) {
        float* at = a.stream_out + static_cast<size_t>(r) * a.outs + feature;
        if (quads && feature < a.outs) {      // (then feature + 3 < outs: the features of a quad exist together)
          float4 s = held[rt];
          s.x += rounded<bf16_t>(acc[rt][0]);
          s.y += rounded<bf16_t>(acc[rt][1]);
          s.z += rounded<bf16_t>(acc[rt][2]);
          s.w += rounded<bf16_t>(acc[rt][3]);
          *reinterpret_cast<float4*>(at) = s;
          squares = s.x * s.x + s.y * s.y + s.z * s.z + s.w * s.w;
          if (a.rows_out != nullptr) {
            const float4 w = gain_held[rt];
            store4<bf16_t>(a.rows_out + static_cast<size_t>(r) * a.outs + feature, floatx4{s.x * w.x, s.y * w.y, s.z * w.z, s.w * w.w});
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (feature + i < a.outs) {
              const float s = at[i] + rounded<bf16_t>(acc[rt][i]);
              at[i] = s;
              squares += s * s;
              if (a.rows_out != nullptr) a.rows_out[static_cast<size_t>(r) * a.outs + feature + i] = from_float<bf16_t>(s * a.gain_out[feature + i]);
            }
        }
      }
      squares += __shfl_xor(squares, 16, kWave);
      squares += __shfl_xor(squares, 32, kWave);
      if (g == 0) a.sums_out[tile * 16 + r] = squares;
    }
  } else if constexpr (GATED) {
    store_tile<bf16_t>(a.y, silu_times(acc[0], acc[1]), r, (row_tile >> 1) * 16 + g * 4, a.rows, a.outs);
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
      if (row_tile + rt < a.n_tiles) store_tile<bf16_t>(a.y, acc[rt], r, (row_tile + rt) * 16 + g * 4, a.rows, a.outs);
  }
}

struct DecodePlan {
  int k_split, waves, blocks;   // parts of k; waves (units) per block; blocks
  bool straddles;               // wave-rows may have their parts of k in two blocks
  double work;                  // bytes' worth of work on the busiest compute unit
};

// How a product is cut into blocks.  `rt`: row tiles per wave; `normed_rows`: rows that every block norms for itself
// (a SCALED product), else 0; `may_straddle`: the caller brought memory for wave-rows whose parts lie in two blocks.
DecodePlan plan_decode(int rt, int n_tiles, int k_tiles, int k, int normed_rows, bool may_straddle) {
  // as many waves as the skinny kernel takes: k is split over the waves of a block while the row tiles are few
  const int wave_rows = (n_tiles + rt - 1) / rt;
  int k_split = 1;
  while (k_split < 8) {
    const int waves_now = wave_rows * k_split, part_after = k_tiles / (k_split * 2);
    if (!((waves_now < 1536 && part_after >= 4) || (waves_now < 2048 && part_after >= 4 * kGroup))) break;
    k_split *= 2;
  }
  // Waves per block.  The compute units share the memory system evenly, so the product is over when the unit with
  // the most bytes is: the number of waves a block gets is chosen for the least work on the busiest unit - its blocks'
  // units (768 wave-rows of 4 parts: 12 waves a block make 256 blocks, one a unit; 8 waves, 384 blocks, would leave
  // half the units with two) and, where blocks norm rows, those rows (counted at 1.5 times their bytes: measured,
  // norming 64 KB of rows costs a block what streaming 90 KB of weights does).  A unit holds as many blocks at once as
  // its 160 KB of LDS and its 32 waves allow; blocks beyond that wait for a further round.  Blocks need not hold
  // whole wave-rows: 320 wave-rows of 8 parts are 256 blocks of 10 waves, one and a quarter wave-rows each - the price
  // is the exchange of one wave-row's sums between two blocks, counted as 96 KB (measured: q/k/v of 6,144 x 4,096 gains
  // nothing from it, o of 5,120 x 8,192 goes from 26 to 20 us, down of 5,120 x 25,600 from 62 to 48).
  constexpr int kMostWaves = 12;
  const DeviceFacts device = device_facts();
  const int kUnits = device.compute_units;
  const size_t kMaxLds = device.lds_bytes;
  const size_t rows_bytes = normed_rows ? static_cast<size_t>(normed_rows) * k * 2 + (12 * 16 + 16) * 4 : 0;
  const double unit_bytes = static_cast<double>(rt) * ((k_tiles + k_split - 1) / k_split) * 1024;
  const double norm_bytes = 1.5 * normed_rows * k * 2, exchange_bytes = 96.0 * 1024;
  const int units = wave_rows * k_split;
  DecodePlan plan{k_split, k_split, 0, false, 0.0};
  for (int waves = k_split; waves <= kMostWaves; ++waves) {
    const bool whole = waves % k_split == 0;
    if (!whole && (!may_straddle || k_split == 1)) continue;
    const int blocks = whole ? (wave_rows + waves / k_split - 1) / (waves / k_split) : (units + waves - 1) / waves;
    const size_t lds = max(rows_bytes, k_split > 1 ? static_cast<size_t>(waves) * rt * 1024 : 0);
    const int at_once = max(1, min(static_cast<int>(lds ? kMaxLds / lds : 32), 32 / waves));
    int on_busiest = (blocks + kUnits - 1) / kUnits;                     // blocks of the unit with the most
    if (on_busiest > at_once) on_busiest = (on_busiest + at_once - 1) / at_once * at_once;   // whole rounds
    const double work = on_busiest * (waves * unit_bytes + norm_bytes) + (whole ? 0.0 : exchange_bytes);
    if (plan.work == 0.0 || work < plan.work) plan = DecodePlan{k_split, waves, blocks, !whole, work};
  }
  if (!normed_rows && plan.waves < 4) {   // blocks of at least 4 waves
    plan.waves = 4;
    plan.blocks = (wave_rows + 4 / k_split - 1) / (4 / k_split);
    plan.straddles = false;
  }
  return plan;
}

template <int RT, bool GATED, bool SCALED, bool ADDS, bool ROWSCALED = false>
int launch_decode(DecodeArgs a, hipStream_t stream) {
  const DecodePlan plan = plan_decode(RT, a.n_tiles, a.k_tiles, a.k, SCALED ? a.rows : 0, a.pieces != nullptr);
  const int k_split = plan.k_split, waves = plan.waves, blocks = plan.blocks;
  a.k_split = k_split;
  a.red_floats = k_split > 1 ? waves * RT * 4 * 64 : 0;
  const size_t lds = max(static_cast<size_t>(a.red_floats) * 4,
                         SCALED ? (12 * 16 + 16) * 4 + static_cast<size_t>(a.rows) * a.k * 2 : (ROWSCALED ? (12 * 16 + 16) * 4 : 0));
  const size_t kMaxLds = device_facts().lds_bytes;
  if (lds > kMaxLds) return -2;
  if (lds > 64 * 1024) {   // more than a block may have without asking: asked once per kernel and device
    static std::mutex guard;
    static bool asked[64] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return -2;
    std::lock_guard<std::mutex> lock(guard);
    if (!asked[device]) {
      const hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_decode_kernel<RT, GATED, SCALED, ADDS, ROWSCALED>),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds));
      if (status != hipSuccess) return static_cast<int>(status);
      asked[device] = true;
    }
  }
  linear_decode_kernel<RT, GATED, SCALED, ADDS, ROWSCALED><<<blocks, waves * 64, lds, stream>>>(a);
  return AKV_LAUNCH_STATUS();
}

}  // namespace

// stream_out [rows, outs] += bfloat16(x W^T (+ bias)) in place (float32; `bias` [outs] float32 or null); sums_out [n_tiles][16] receives, for every row tile of
// 16 outputs and every row, the sum of squares of the new values (rows beyond `rows`: 0).  rows <= 16, k % 8 == 0.
// `pieces` (exchange_tiles * 512 floats) and `arrivals` (exchange_tiles words, zero; left zero) may be null, or hold
// fewer than n_tiles + 1 row tiles' worth (a wave's pair of row tiles may begin at the last tile), and are then not used: with them the product
// may be cut into blocks that do not hold whole row tiles' parts of k (see plan_decode).  Launches that share them
// follow each other on one stream.
// What plan_decode makes of a product (for tests and measurements): out[0..4] = parts of k, waves per block, blocks,
// whether row tiles may have their parts of k in two blocks, the busiest compute unit's work in KB.
extern "C" int akv_linear_decode_plan(int rt, int n_tiles, int k_tiles, int k, int normed_rows, int may_straddle, int* out) {
  const DecodePlan plan = plan_decode(rt, n_tiles, k_tiles, k, normed_rows, may_straddle != 0);
  out[0] = plan.k_split, out[1] = plan.waves, out[2] = plan.blocks, out[3] = plan.straddles ? 1 : 0;
  out[4] = static_cast<int>(plan.work / 1024.0);
  return 0;
}

namespace {
int linear_adds(const void* x, const void* wp, float* stream_out, float* sums_out, float* pieces,
                unsigned int* arrivals, int exchange_tiles, int rows, int outs, int k, int n_tiles,
                int k_tiles, const float* bias, void* rows_out, const float* gain, hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if (rows > 16 || (k & 7) != 0 || n_tiles * 16 < outs || (n_tiles - 1) * 16 >= outs || k_tiles * 32 < k) return -2;
  if ((rows_out == nullptr) != (gain == nullptr)) return -2;
  DecodeArgs a{};
  a.x = static_cast<const bf16_t*>(x);
  a.wp = static_cast<const uintx4*>(wp);
  a.stream_out = stream_out;
  a.sums_out = sums_out;
  a.rows_out = static_cast<bf16_t*>(rows_out);
  a.gain_out = gain;
  a.bias = bias;
  if (pieces != nullptr && arrivals != nullptr && exchange_tiles >= n_tiles + 1) a.pieces = pieces, a.arrivals = arrivals;
  a.rows = rows, a.outs = outs, a.k = k, a.k_tiles = k_tiles, a.n_tiles = n_tiles;
  return launch_decode<1, false, false, true>(a, stream);
}
}  // namespace

extern "C" int akv_linear_adds(const void* x, const void* wp, float* stream_out, float* sums_out, float* pieces,
                               unsigned int* arrivals, int exchange_tiles, int rows, int outs, int k, int n_tiles,
                               int k_tiles, const float* bias, hipStream_t stream) {
  return linear_adds(x, wp, stream_out, sums_out, pieces, arrivals, exchange_tiles, rows, outs, k, n_tiles, k_tiles, bias,
                     nullptr, nullptr, stream);
}

// The same, and rows_out [rows, outs] bfloat16 receives the new residual sum times `gain` [outs] (the weight of the
// norm that follows): what akv_linear_rowscaled reads.
extern "C" int akv_linear_adds_rows(const void* x, const void* wp, float* stream_out, float* sums_out, float* pieces,
                                    unsigned int* arrivals, int exchange_tiles, int rows, int outs, int k, int n_tiles,
                                    int k_tiles, const float* bias, void* rows_out, const float* gain, hipStream_t stream) {
  if (rows_out == nullptr || gain == nullptr) return -2;
  return linear_adds(x, wp, stream_out, sums_out, pieces, arrivals, exchange_tiles, rows, outs, k, n_tiles, k_tiles, bias,
                     rows_out, gain, stream);
}

// y [rows, outs] = (x W^T) with every row scaled by rsqrt(its mean of squares + eps), plus `bias` (gated: silu of
// the scaled gate times the scaled up): x [rows, k] bfloat16 are the rows akv_linear_adds_rows left - the residual
// sum times the norm's weight -, `sums` [sum_tiles][16] the partial sums of squares of the residual rows it left
// (sum_tiles = ceil(k / 16)).  Sizes, `pieces`, `arrivals`, `row_tiles`: as for akv_linear_scaled, without its limit
// on the rows' bytes.
extern "C" int akv_linear_rowscaled(const void* x, const float* sums, int sum_tiles, float eps, const void* wp, void* y,
                                    float* pieces, unsigned int* arrivals, int exchange_tiles, int rows, int outs, int k,
                                    int n_tiles, int k_tiles, int gated, int row_tiles, const float* bias,
                                    hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if (rows > 16 || (k & 7) != 0 || k_tiles * 32 < k || sum_tiles != (k + 15) / 16) return -2;
  if (row_tiles < 0 || row_tiles > 2 || (gated && (row_tiles == 1 || bias != nullptr))) return -2;
  if (gated ? ((outs & 15) != 0 || n_tiles * 8 != outs) : n_tiles * 16 < outs) return -2;
  DecodeArgs a{};
  a.x = static_cast<const bf16_t*>(x);
  a.sums = sums;
  a.sum_tiles = sum_tiles;
  a.eps = eps;
  a.wp = static_cast<const uintx4*>(wp);
  a.y = static_cast<bf16_t*>(y);
  a.bias = bias;
  if (pieces != nullptr && arrivals != nullptr && exchange_tiles >= n_tiles + 1) a.pieces = pieces, a.arrivals = arrivals;
  const bool may = a.pieces != nullptr;
  a.rows = rows, a.outs = outs, a.k = k, a.k_tiles = k_tiles, a.n_tiles = n_tiles;
  if (gated) return launch_decode<2, true, false, false, true>(a, stream);
  // (rows from memory: two row tiles a wave share the rows' loads, as in the plain product)
  if (row_tiles == 0)
    row_tiles = n_tiles >= 2 && plan_decode(2, n_tiles, k_tiles, k, 0, may).work < plan_decode(1, n_tiles, k_tiles, k, 0, may).work ? 2 : 1;
  if (row_tiles == 2) return launch_decode<2, false, false, false, true>(a, stream);
  return launch_decode<1, false, false, false, true>(a, stream);
}

// y [rows, outs] = norm(stream) W^T (gated: y [rows, inter] = silu(. Wgate^T) * (. Wup^T), wp as for
// akv_linear_packed_swiglu), where norm(stream) is what akv_add_rmsnorm gives for the float32 rows `stream` [rows, k]
// and the weight `gain` [k] - with the rows' sums of squares not formed here but taken from `sums`
// [sum_tiles][16] (what akv_linear_adds left: sum_tiles = ceil(k / 16)).  rows <= 16, k % 8 == 0, and the normed rows
// (rows * k bfloat16) fit into a compute unit's LDS (160 KB) beside 832 bytes; -2 otherwise.  `pieces`, `arrivals`: as
// for akv_linear_adds.  `row_tiles`: row tiles per wave of the plain product, 1 or 2; 0 leaves the choice to the sizes (a
// gated product's waves always take a pair).  `bias` [outs] float32 or null (never with `gated`): y = norm(stream) W^T + bias.
extern "C" int akv_linear_scaled(const float* stream_in, const float* sums, int sum_tiles, const float* gain, float eps,
                                 const void* wp, void* y, float* pieces, unsigned int* arrivals, int exchange_tiles,
                                 int rows, int outs, int k, int n_tiles, int k_tiles, int gated, int row_tiles,
                                 const float* bias, hipStream_t stream) {
  if (rows <= 0 || outs <= 0) return 0;
  if (rows > 16 || (k & 7) != 0 || k_tiles * 32 < k || sum_tiles != (k + 15) / 16) return -2;
  if (row_tiles < 0 || row_tiles > 2 || (gated && (row_tiles == 1 || bias != nullptr))) return -2;
  if (gated ? ((outs & 15) != 0 || n_tiles * 8 != outs) : n_tiles * 16 < outs) return -2;
  DecodeArgs a{};
  a.stream = stream_in;
  a.sums = sums;
  a.sum_tiles = sum_tiles;
  a.gain = gain;
  a.eps = eps;
  a.wp = static_cast<const uintx4*>(wp);
  a.y = static_cast<bf16_t*>(y);
  a.bias = bias;
  if (pieces != nullptr && arrivals != nullptr && exchange_tiles >= n_tiles + 1) a.pieces = pieces, a.arrivals = arrivals;
  const bool may = a.pieces != nullptr;
  a.rows = rows, a.outs = outs, a.k = k, a.k_tiles = k_tiles, a.n_tiles = n_tiles;
  if (gated) return launch_decode<2, true, true, false>(a, stream);
  // The rows come from LDS, so two row tiles per wave save no loads of activations; they are two runs of memory per
  // wave where one is faster (q/k/v at 4 rows: 19.4 -> 16.3 us, at 8: 20.3 -> 19.4; counted as 1.3 times the bytes, which puts the rule where the measurements are).
  // They pay where the normed rows fill so much LDS that a compute unit holds one block, and the blocks of one row tile
  // per wave would need a second round (16 rows of 4,096: 28.8 -> 23.0 us).
  if (row_tiles == 0)
    row_tiles = n_tiles >= 2 && plan_decode(2, n_tiles, k_tiles, k, rows, may).work * 1.3 < plan_decode(1, n_tiles, k_tiles, k, rows, may).work ? 2 : 1;
  if (row_tiles == 2) return launch_decode<2, false, true, false>(a, stream);
  return launch_decode<1, false, true, false>(a, stream);
}
