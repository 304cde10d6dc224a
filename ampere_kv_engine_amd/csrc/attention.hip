// Attention over the paged cache.
//
// `attention_rows` is the plain path (all of float32, and bfloat16 until a faster kernel takes a case): one
// wave per (token, query head).  Keys are visited in tiles of 64 aligned to absolute key positions, so the
// order of every sum depends on the token's own position only - not on how the request was cut into steps or
// on what else is in the batch.  Scores, softmax and the weighted sum are float32; query head h reads kv head
// h / (q_heads / kv_heads); a query at position p sees keys max(0, p - window + 1) .. p of its own request
// (ampere_kv/kv_cache.py:80-94 for group mapping, scale and mask; split softmax as in csrc/paged_decode.cu:182-236).

#include "common.h"
#include "api.h"

using namespace akv;

namespace {

constexpr int kMaxDimRegs = 4;  // head dims up to 256: each lane owns dims lane, lane + 64, ...

__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T>
__global__ __launch_bounds__(256) void attention_rows_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, const int* __restrict__ block_table,
    const int* __restrict__ table_rows, int table_width, T* __restrict__ out, long tokens, int q_heads, int kv_heads, int dim, int page_size,
    long num_pages, float scale, int window) {
  extern __shared__ unsigned char lds_raw[];
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const long row = static_cast<long>(blockIdx.x) * waves + wave;
  if (row >= tokens * q_heads) return;
  // per wave: dim floats of q, 64 weights, 64 value-row offsets
  const size_t per_wave = static_cast<size_t>(dim) * 4 + kWave * 4 + kWave * 8;
  float* qs = reinterpret_cast<float*>(lds_raw + wave * per_wave);
  float* ps = qs + dim;
  long* offs = reinterpret_cast<long*>(ps + kWave);

  const long n = row / q_heads;
  const int h = static_cast<int>(row % q_heads);
  const int kvh = h / (q_heads / kv_heads);
  const int r = table_rows != nullptr ? table_rows[seq_of_token[n]] : seq_of_token[n];   // the table's row of the request
  const int pos = positions[n];
  const int lowest = window > 0 ? max(0, pos - window + 1) : 0;
  for (int i = lane; i < dim; i += kWave) qs[i] = to_float(q[row * dim + i]);
  wave_sync_lds();

  float m = -INFINITY, l = 0.f;
  float acc[kMaxDimRegs] = {0.f, 0.f, 0.f, 0.f};
  for (int tile = lowest / kWave; tile * kWave <= pos; ++tile) {
    const int j = tile * kWave + lane;
    const bool valid = j >= lowest && j <= pos;
    float s = -INFINITY;
    long value_at = -1;
    if (valid) {
      const long page = block_table[static_cast<long>(r) * table_width + j / page_size];
      if (page < 0 || page >= num_pages) {
        s = __uint_as_float(0x7fc00000u);  // a page that is not the request's: poison, never read
      } else {
        const T* kp = k_pages + ((page * kv_heads + kvh) * page_size + j % page_size) * dim;
        float dot = 0.f;
        for (int i = 0; i < dim; ++i) dot = fmaf(qs[i], to_float(kp[i]), dot);
        s = dot * scale;
        value_at = (page * kv_heads + kvh) * dim * page_size + j % page_size;  // values are [dim, page_size]
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float correction = expf(m - m_new);
    l = l * correction + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    offs[lane] = value_at;
    wave_sync_lds();
#pragma unroll
    for (int c = 0; c < kMaxDimRegs; ++c) acc[c] *= correction;
    for (int jj = 0; jj < kWave; ++jj) {
      const long at = offs[jj];
      if (at < 0) continue;  // uniform over the wave
      const float pj = ps[jj];
#pragma unroll
      for (int c = 0; c < kMaxDimRegs; ++c) {
        const int i = lane + c * kWave;
        if (i < dim) acc[c] = fmaf(pj, to_float(v_pages[at + static_cast<long>(i) * page_size]), acc[c]);
      }
    }
    wave_sync_lds();
  }
#pragma unroll
  for (int c = 0; c < kMaxDimRegs; ++c) {
    const int i = lane + c * kWave;
    if (i < dim) out[row * dim + i] = from_float<T>(acc[c] / l);
  }
}

}  // namespace

// ---- the cut of single tokens' keys for the matrix-core decode attention ----------------------------------------------
// The decode attention works on (request, segment of its keys) items.  Segments have ONE size for all requests of a
// launch, worked out here from the lengths on the device: a long request among short ones gets as many segments as its
// keys need, no block is started for a segment that holds nothing, and a step that was recorded once and is replayed
// with other lengths is cut as the same step run eagerly would be.  One wave; lane r looks at request seq_first + r
// (at most 64).  A request's keys span from `first` (the start of its window, down to a multiple of 32) to its token's
// position; the size is the sum of the spans over items_wanted, up to a multiple of 32, at least min_segment; items
// are numbered request by request.  The cut depends on the lengths only, so one plan serves every layer of a step.
//   plan[0] = items in all, plan[1] = keys per segment
//   plan[4 + 2 r] = items before request r's, plan[5 + 2 r] = its items                          (r < 64)
//   plan[132 + 4 i] = request of item i (counted from seq_first), its first key, the token's position, its last key
namespace {
__global__ __launch_bounds__(64) void decode_plan_kernel(const int* __restrict__ seq_lens, int seq_first, int seq_count,
                                                        int window, int items_wanted, int min_segment, int items_grid,
                                                        int* __restrict__ plan) {
  const int lane = threadIdx.x;
  int pos = -1, first = 0, span = 0;
  if (lane < seq_count) {
    pos = seq_lens[seq_first + lane] - 1;
    first = (window > 0 ? max(0, pos - window + 1) : 0) & ~31;
    span = max(pos - first + 1, 0);
  }
  int total_span = span;
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) total_span += __shfl_xor(total_span, offset, kWave);
  const int size = max(min_segment, ((total_span + items_wanted - 1) / items_wanted + 31) & ~31);
  const int count = (span + size - 1) / size;
  int upto = count;  // inclusive prefix sum over the wave
#pragma unroll
  for (int step = 1; step < kWave; step <<= 1) {
    const int other = __shfl_up(upto, step, kWave);
    if (lane >= step) upto += other;
  }
  const int before = upto - count;
  if (lane == kWave - 1) {
    plan[0] = min(upto, items_grid);
    plan[1] = size;
  }
  plan[4 + 2 * lane] = before;
  plan[5 + 2 * lane] = count;
  for (int z = 0; z < count; ++z) {
    const int item = before + z;
    if (item >= items_grid) break;  // (cannot happen with the host's bound; never write beyond the buffer)
    const int lo = first + z * size;
    *reinterpret_cast<int4*>(plan + 132 + 4 * item) = make_int4(lane, lo, pos, min(pos, lo + size - 1));
  }
}
}  // namespace

extern "C" int akv_decode_plan(const int* seq_lens, int seq_first, int seq_count, int window, int items_wanted,
                               int min_segment, int items_grid, int* plan, hipStream_t stream) {
  if (seq_count <= 0) return 0;
  if (seq_count > 64 || items_wanted < 1 || min_segment < 32 || (min_segment & 31) != 0 || items_grid < 1) return -2;
  decode_plan_kernel<<<1, 64, 0, stream>>>(seq_lens, seq_first, seq_count, window, items_wanted, min_segment, items_grid,
                                           plan);
  return AKV_LAUNCH_STATUS();
}

extern "C" int akv_attention_rows(const void* q, const void* k_pages, const void* v_pages, const int* seq_of_token,
                                  const int* positions, const int* block_table, const int* table_rows, int table_width,
                                  void* out, int dtype,
                                  long tokens, int q_heads, int kv_heads, int dim, int page_size, long num_pages,
                                  float scale, int window, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (dim > kMaxDimRegs * kWave || q_heads % kv_heads != 0) return -2;
  const long rows = tokens * q_heads;
  const size_t lds = 4 * (static_cast<size_t>(dim) * 4 + kWave * 4 + kWave * 8);
  AKV_DISPATCH(dtype, T,
               attention_rows_kernel<T><<<static_cast<unsigned>((rows + 3) / 4), 256, lds, stream>>>(
                   static_cast<const T*>(q), static_cast<const T*>(k_pages), static_cast<const T*>(v_pages),
                   seq_of_token, positions, block_table, table_rows, table_width, static_cast<T*>(out), tokens, q_heads,
                   kv_heads,
                   dim, page_size, num_pages, scale, window));
  return AKV_LAUNCH_STATUS();
}
