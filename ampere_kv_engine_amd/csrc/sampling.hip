// Choosing the next token from float32 logits.
//   temperature == 0: the largest logit, ties to the lowest id (the reference's argmax, ampere_kv/runner.py:346).
//   temperature  > 0: a draw from softmax(logits / temperature) by the Gumbel-max rule:
//                     argmax_i( logits[i] / temperature - log(-log(u_i)) ), u_i uniform in (0, 1).
// u_i comes from Philox-4x32-10 keyed by the request's seed with counter (i, draw number), so a request's draws
// depend on its own seed and draw count only, never on the batch it shares a step with.
// A row that holds a NaN, or no logit above -infinity, has no next token: the result is -1 (the attention kernels
// answer a block table that names a page outside the pool with NaN, and that must not turn into token 0).

#include "common.h"
#include "api.h"

using namespace akv;

namespace {

__device__ __forceinline__ uint32_t philox_first(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1) {
  uint32_t c2 = 0u, c3 = 0u;
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * c0;
    const uint64_t p1 = static_cast<uint64_t>(0xCD9E8D57u) * c2;
    const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = static_cast<uint32_t>(p1);
    const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = static_cast<uint32_t>(p0);
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

// SLOTS: the sampling state is not handed in row by row but read from (and written to) the slot of the row's request:
// the row's token row is rows_of[row], its request seq_of_token[...], its slot seq_slots[...]; slot words 2..5 hold
// temperature, seed and draws made so far, word 1 receives the chosen token and word 5 counts the draw (the words are
// named in common.h).

template <bool SLOTS>
__global__ __launch_bounds__(1024) void sample_kernel(const float* __restrict__ logits,
                                                      const float* __restrict__ temperature,
                                                      const unsigned long long* __restrict__ seeds,
                                                      const unsigned int* __restrict__ draws, int* __restrict__ out,
                                                      int vocab, const int* __restrict__ rows_of,
                                                      const int* __restrict__ seq_of_token,
                                                      const int* __restrict__ seq_slots, int* __restrict__ slot_words) {
  __shared__ float best_value[16];
  __shared__ int best_index[16];
  __shared__ int any_nan;
  if (threadIdx.x == 0) any_nan = 0;
  __syncthreads();
  bool saw_nan = false;
  const int row = blockIdx.x;
  const float* x = logits + static_cast<size_t>(row) * vocab;
  float t;
  uint32_t k0, k1, draw;
  int* words = nullptr;
  if constexpr (SLOTS) {
    words = slot_words + static_cast<size_t>(seq_slots[seq_of_token[rows_of[row]]]) * kSlotWords;
    t = __int_as_float(words[kSlotTemperature]);
    k0 = static_cast<uint32_t>(words[kSlotSeedLow]);
    k1 = static_cast<uint32_t>(words[kSlotSeedHigh]);
    draw = static_cast<uint32_t>(words[kSlotDraws]);
    __syncthreads();   // every thread has read the state before thread 0 writes it below
  } else {
    t = temperature != nullptr ? temperature[row] : 0.f;
    k0 = t > 0.f ? static_cast<uint32_t>(seeds[row]) : 0u;
    k1 = t > 0.f ? static_cast<uint32_t>(seeds[row] >> 32) : 0u;
    draw = t > 0.f ? draws[row] : 0u;
  }
  float value = -INFINITY;
  int index = vocab;  // "none yet"; any real index is lower
  // eight loads of a thread are on their way before the first is looked at; ids still ascend per thread, so the
  // first maximum stays.  (Every load is issued whatever its place - beyond the row it asks for the row's last piece,
  // which is then not looked at -: behind a test each, the eight would be waited for one by one.)
  constexpr int kAhead = 8;
  auto look_at = [&](int i, float score) {
    saw_nan |= score != score;
    if (t > 0.f && i < vocab) {
      const uint32_t bits = philox_first(static_cast<uint32_t>(i), draw, k0, k1);
      const float u01 = (static_cast<float>(bits >> 8) + 0.5f) * 0x1p-24f;
      score = score / t - logf(-logf(u01));
    }
    if (i < vocab && score > value) { value = score; index = i; }
  };
  if ((vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
    // rows of whole 16-byte pieces: a thread takes four consecutive ids a load (a row of 151,936 logits is 19 trips
    // to memory with single loads, 5 with these)
    const int pieces = vocab / 4;
    for (int p0 = threadIdx.x; p0 < pieces; p0 += kAhead * blockDim.x) {
      float4 fetched[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int p = min(p0 + u * static_cast<int>(blockDim.x), pieces - 1);
        fetched[u] = *reinterpret_cast<const float4*>(x + 4 * static_cast<size_t>(p));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int i = 4 * (p0 + u * blockDim.x);
        if (i < vocab) {
          look_at(i, fetched[u].x);
          look_at(i + 1, fetched[u].y);
          look_at(i + 2, fetched[u].z);
          look_at(i + 3, fetched[u].w);
        }
      }
    }
  } else {
    for (int i0 = threadIdx.x; i0 < vocab; i0 += kAhead * blockDim.x) {
      float fetched[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        fetched[u] = x[min(i0 + u * static_cast<int>(blockDim.x), vocab - 1)];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kAhead; ++u) look_at(i0 + u * blockDim.x, fetched[u]);
    }
  }
  for (int offset = kWave / 2; offset > 0; offset >>= 1) {
    const float other_value = __shfl_xor(value, offset, kWave);
    const int other_index = __shfl_xor(index, offset, kWave);
    if (other_value > value || (other_value == value && other_index < index)) { value = other_value; index = other_index; }
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) { best_value[wave] = value; best_index[wave] = index; }
  if (__any(saw_nan) && lane == 0) any_nan = 1;      // (every writer stores the same value)
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < blockDim.x / kWave; ++w)
      if (best_value[w] > value || (best_value[w] == value && best_index[w] < index)) { value = best_value[w]; index = best_index[w]; }
    const int token = (index < vocab && any_nan == 0) ? index : -1;
    out[row] = token;
    if constexpr (SLOTS) {
      words[kSlotLastToken] = token;
      words[kSlotDraws] = static_cast<int>(draw + 1u);
    }
  }
}

// The same choice with a row's ids cut over `parts` blocks (a block on one compute unit draws a fraction of what the
// device can: a row of 151,936 logits takes one block 18 us).  Block (row, part) scans its run of ids and leaves its
// best (value, id; id -2: it saw a NaN) in `part_values` / `part_ids` [rows][parts]; `arrivals` [rows] (zero between
// launches) tells the last block of a row, which picks the best of the parts - the largest value, the lowest id
// among equals: the choice does not depend on the cut or on who is last - and writes the token and the slot.
// parts <= 64; SLOTS as above: every block reads the row's state before it arrives, the last writes it.
template <bool SLOTS>
__global__ __launch_bounds__(256) void sample_parts_kernel(const float* __restrict__ logits,
                                                           const float* __restrict__ temperature,
                                                           const unsigned long long* __restrict__ seeds,
                                                           const unsigned int* __restrict__ draws, int* __restrict__ out,
                                                           int vocab, const int* __restrict__ rows_of,
                                                           const int* __restrict__ seq_of_token,
                                                           const int* __restrict__ seq_slots, int* __restrict__ slot_words,
                                                           int parts, float* __restrict__ part_values,
                                                           int* __restrict__ part_ids, unsigned int* __restrict__ arrivals) {
  __shared__ float best_value[4];
  __shared__ int best_index[4];
  __shared__ int any_nan, is_last;
  if (threadIdx.x == 0) any_nan = 0;
  __syncthreads();
  bool saw_nan = false;
  const int row = blockIdx.x / parts, part = blockIdx.x % parts;
  const float* x = logits + static_cast<size_t>(row) * vocab;
  float t;
  uint32_t k0, k1, draw;
  int* words = nullptr;
  if constexpr (SLOTS) {
    words = slot_words + static_cast<size_t>(seq_slots[seq_of_token[rows_of[row]]]) * kSlotWords;
    t = __int_as_float(words[kSlotTemperature]);
    k0 = static_cast<uint32_t>(words[kSlotSeedLow]);
    k1 = static_cast<uint32_t>(words[kSlotSeedHigh]);
    draw = static_cast<uint32_t>(words[kSlotDraws]);
  } else {
    t = temperature != nullptr ? temperature[row] : 0.f;
    k0 = t > 0.f ? static_cast<uint32_t>(seeds[row]) : 0u;
    k1 = t > 0.f ? static_cast<uint32_t>(seeds[row] >> 32) : 0u;
    draw = t > 0.f ? draws[row] : 0u;
  }
  float value = -INFINITY;
  int index = vocab;  // "none yet"; any real index is lower
  constexpr int kAhead = 8;
  auto look_at = [&](int i, float score) {
    saw_nan |= score != score;
    if (t > 0.f) {
      const uint32_t bits = philox_first(static_cast<uint32_t>(i), draw, k0, k1);
      const float u01 = (static_cast<float>(bits >> 8) + 0.5f) * 0x1p-24f;
      score = score / t - logf(-logf(u01));
    }
    if (score > value) { value = score; index = i; }
  };
  if ((vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
    const int pieces = vocab / 4, per = (pieces + parts - 1) / parts;
    const int begin = part * per, end = min(pieces, begin + per);
    for (int p0 = begin + threadIdx.x; p0 < end; p0 += kAhead * blockDim.x) {
      float4 fetched[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u)
        fetched[u] = *reinterpret_cast<const float4*>(x + 4 * static_cast<size_t>(min(p0 + u * static_cast<int>(blockDim.x), end - 1)));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int p = p0 + u * blockDim.x;
        if (p < end) {
          look_at(4 * p, fetched[u].x);
          look_at(4 * p + 1, fetched[u].y);
          look_at(4 * p + 2, fetched[u].z);
          look_at(4 * p + 3, fetched[u].w);
        }
      }
    }
  } else {
    const int per = (vocab + parts - 1) / parts;
    const int begin = part * per, end = min(vocab, begin + per);
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += kAhead * blockDim.x) {
      float fetched[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) fetched[u] = x[min(i0 + u * static_cast<int>(blockDim.x), end - 1)];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kAhead; ++u)
        if (i0 + u * static_cast<int>(blockDim.x) < end) look_at(i0 + u * blockDim.x, fetched[u]);
    }
  }
  auto better = [](float other_value, int other_index, float& value, int& index) {
    if (other_value > value || (other_value == value && other_index < index)) { value = other_value; index = other_index; }
  };
  for (int offset = kWave / 2; offset > 0; offset >>= 1) better(__shfl_xor(value, offset, kWave), __shfl_xor(index, offset, kWave), value, index);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) { best_value[wave] = value; best_index[wave] = index; }
  if (__any(saw_nan) && lane == 0) any_nan = 1;      // (every writer stores the same value)
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < static_cast<int>(blockDim.x) / kWave; ++w) better(best_value[w], best_index[w], value, index);
    publish(part_values + static_cast<size_t>(row) * parts + part, value);
    __hip_atomic_store(part_ids + static_cast<size_t>(row) * parts + part, any_nan != 0 ? -2 : index, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    is_last = arrive(arrivals + row) == static_cast<unsigned>(parts - 1) ? 1 : 0;
  }
  __syncthreads();
  if (is_last == 0 || wave != 0) return;
  // the row's last block: lane p takes part p
  value = -INFINITY, index = vocab;
  bool nan_seen = false;
  if (lane < parts) {
    value = collect(part_values + static_cast<size_t>(row) * parts + lane);
    index = __hip_atomic_load(part_ids + static_cast<size_t>(row) * parts + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    nan_seen = index == -2;
    if (nan_seen) value = -INFINITY, index = vocab;
  }
  nan_seen = __any(nan_seen);
  for (int offset = kWave / 2; offset > 0; offset >>= 1) better(__shfl_xor(value, offset, kWave), __shfl_xor(index, offset, kWave), value, index);
  if (lane == 0) {
    __hip_atomic_store(arrivals + row, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
    const int token = (index < vocab && !nan_seen) ? index : -1;
    out[row] = token;
    if constexpr (SLOTS) {
      words[kSlotLastToken] = token;
      words[kSlotDraws] = static_cast<int>(draw + 1u);
    }
  }
}

}  // namespace

// `parts` blocks a row (2..64) through the workspace `part_values`, `part_ids` ([rows][parts] each) and `arrivals`
// ([rows], zero before the first launch; left zero): see sample_parts_kernel.  Launches that share the workspace
// follow each other on one stream.
extern "C" int akv_sample_parts(const float* logits, const float* temperature, const unsigned long long* seeds,
                                const unsigned int* draws, const int* rows_of, const int* seq_of_token,
                                const int* seq_slots, int* slot_words, int* out, int rows, int vocab, int parts,
                                float* part_values, int* part_ids, unsigned int* arrivals, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (parts < 2 || parts > 64 || part_values == nullptr || part_ids == nullptr || arrivals == nullptr) return -2;
  if (static_cast<long>(rows) * parts > 0x7fffffffL) return -2;
  if (slot_words != nullptr)
    sample_parts_kernel<true><<<rows * parts, 256, 0, stream>>>(logits, nullptr, nullptr, nullptr, out, vocab, rows_of, seq_of_token,
                                                                seq_slots, slot_words, parts, part_values, part_ids, arrivals);
  else
    sample_parts_kernel<false><<<rows * parts, 256, 0, stream>>>(logits, temperature, seeds, draws, out, vocab, nullptr, nullptr,
                                                                 nullptr, nullptr, parts, part_values, part_ids, arrivals);
  return AKV_LAUNCH_STATUS();
}

extern "C" int akv_sample(const float* logits, const float* temperature, const unsigned long long* seeds,
                          const unsigned int* draws, int* out, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  sample_kernel<false><<<rows, 1024, 0, stream>>>(logits, temperature, seeds, draws, out, vocab, nullptr, nullptr, nullptr,
                                                  nullptr);
  return AKV_LAUNCH_STATUS();
}

// The same choice with every row's temperature, seed and draw count read from the slot of its request, where the
// chosen token and the new draw count are left too.  rows_of [rows]: the step's token row that logits row i belongs
// to.  No two rows may belong to one request (they would share a draw count).
extern "C" int akv_sample_slots(const float* logits, const int* rows_of, const int* seq_of_token, const int* seq_slots,
                                int* slot_words, int* out, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  sample_kernel<true><<<rows, 1024, 0, stream>>>(logits, nullptr, nullptr, nullptr, out, vocab, rows_of, seq_of_token,
                                                 seq_slots, slot_words);
  return AKV_LAUNCH_STATUS();
}
