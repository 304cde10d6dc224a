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

}  // namespace

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
