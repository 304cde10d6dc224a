// Token-wise kernels: embedding gather, RMSNorm (alone, with the residual add, per head), rotary encoding,
// cache write, the fused q/k-norm + rotation + cache write, SwiGLU, row gather.
// Statistics, angles and the residual sum are float32 whatever the activation type T is.

#include <type_traits>

#include "common.h"
#include "api.h"

using namespace akv;

namespace {

// ---- per-request state of fixed size: kSlotWords 32-bit words per slot (the words are named in common.h) -----------

// What a step changes in the persistent integer state before its first kernel reads it: `count` (offset, value) pairs
// - block-table entries of pages the step's requests were given or gave back - and the requests' new lengths.
__global__ void step_prologue_kernel(int* __restrict__ state, long state_size, const int* __restrict__ patches,
                                     const int* __restrict__ count, int capacity, const int* __restrict__ seq_slots,
                                     const int* __restrict__ seq_lens, int seqs) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < capacity && i < count[0]) {
    const long at = patches[2 * i];
    if (at >= 0 && at < state_size) state[at] = patches[2 * i + 1];   // (never write outside the state)
  }
  if (i < seqs) {
    const long at = static_cast<long>(seq_slots[i]) * kSlotWords + kSlotLength;
    if (at >= 0 && at < state_size) state[at] = seq_lens[i];
  }
}

// ---- embedding: out[n, :] = table[ids[n], :] widened to float32 (no scaling) ------------------------------
// An id of -1 stands for the token that was chosen last for the row's request (kept in its slot by the sampler).
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out,
                             int hidden, int vocab, const int* __restrict__ seq_of_token,
                             const int* __restrict__ seq_slots, const int* __restrict__ slot_words) {
  const int n = blockIdx.x;
  int id = ids[n];
  if (id == -1 && slot_words != nullptr) id = slot_words[seq_slots[seq_of_token[n]] * kSlotWords + kSlotLastToken];
  float* dst = out + static_cast<size_t>(n) * hidden;
  if (id < 0 || id >= vocab) {  // never read outside the table; a poisoned row shows the fault downstream
    for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = __uint_as_float(0x7fc00000u);
    return;
  }
  const T* src = table + static_cast<size_t>(id) * hidden;
  if constexpr (std::is_same<T, bf16_t>::value) {
    if ((hidden & 7) == 0) {     // 16 bytes of the row a thread and turn, all of a thread's loads on their way at once
      constexpr int kTurns = 4;
      for (int d0 = threadIdx.x * 8; d0 < hidden; d0 += kTurns * blockDim.x * 8) {
        uint4 raw[kTurns];
#pragma unroll
        for (int u = 0; u < kTurns; ++u)
          raw[u] = *reinterpret_cast<const uint4*>(src + min(d0 + u * static_cast<int>(blockDim.x) * 8, hidden - 8));
#pragma unroll
        for (int u = 0; u < kTurns; ++u) {
          const int d = d0 + u * blockDim.x * 8;
          if (d >= hidden) break;
          const uint32_t w[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
          *reinterpret_cast<float4*>(dst + d) = make_float4(__uint_as_float(w[0] << 16), __uint_as_float(w[0] & 0xffff0000u),
                                                            __uint_as_float(w[1] << 16), __uint_as_float(w[1] & 0xffff0000u));
          *reinterpret_cast<float4*>(dst + d + 4) = make_float4(__uint_as_float(w[2] << 16), __uint_as_float(w[2] & 0xffff0000u),
                                                                __uint_as_float(w[3] << 16), __uint_as_float(w[3] & 0xffff0000u));
        }
      }
      return;
    }
  }
  for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = to_float(src[d]);
}

// ---- residual add + RMSNorm: stream += delta (float32); out = T( T(stream * rsqrt(mean^2 + eps)) * w ) ----
// One block per row.  A thread owns groups of 4 consecutive elements (16-byte accesses); a row of up to
// 256 * 4 * GROUPS elements (GROUPS = 4, 8 or 16: rows up to 16,384 wide) stays in registers between the sum of
// squares and the scaling, longer rows are read a second time.

template <typename T> __device__ __forceinline__ float4 load4(const T* p);
template <> __device__ __forceinline__ float4 load4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 load4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                     __uint_as_float(v.y & 0xffff0000u));
}
template <typename T> __device__ __forceinline__ void store4(T* p, float4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float4 v) {
  uint2 packed;
  packed.x = bf16_pair(v.x, v.y);
  packed.y = bf16_pair(v.z, v.w);
  *reinterpret_cast<uint2*>(p) = packed;
}

template <typename T, int GROUPS>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ stream, const T* __restrict__ delta,
                                                          const float* __restrict__ weight, float eps,
                                                          T* __restrict__ out, int hidden) {
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * hidden;
  float* s = stream + base;
  T* o = out + base;
  float acc = 0.f;
  if ((hidden & 3) == 0 && hidden <= 256 * 4 * GROUPS) {
    // Every group's loads go out before anything waits, whatever the row's width (a group beyond the row reads its
    // last four values and counts for nothing): behind a test per group the compiler waits for each group's loads,
    // and for its store, before it asks for the next - eight trips to memory a row instead of one.
    float4 kept[GROUPS], added[GROUPS], gain[GROUPS];
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) kept[j] = load4<float>(s + min((j * 256 + static_cast<int>(threadIdx.x)) * 4, hidden - 4));
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) gain[j] = load4<float>(weight + min((j * 256 + static_cast<int>(threadIdx.x)) * 4, hidden - 4));
    if (delta != nullptr) {   // (last: what is widened to float32 as it arrives is waited for at once)
#pragma unroll
      for (int j = 0; j < GROUPS; ++j) added[j] = load4<T>(delta + base + min((j * 256 + static_cast<int>(threadIdx.x)) * 4, hidden - 4));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) {
      const int i = (j * 256 + threadIdx.x) * 4;
      float4 v = kept[j];
      if (delta != nullptr) {
        const float4 d = added[j];
        v = make_float4(v.x + d.x, v.y + d.y, v.z + d.z, v.w + d.w);
        if (i < hidden) store4<float>(s + i, v);
      }
      kept[j] = v;
      if (i < hidden) acc += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    const float scale = rsqrtf(block_sum(acc, scratch) / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) {
      const int i = (j * 256 + threadIdx.x) * 4;
      if (i < hidden) {
        const float4 v = kept[j], w = gain[j];
        store4<T>(o + i, make_float4(rounded<T>(v.x * scale) * w.x, rounded<T>(v.y * scale) * w.y,
                                     rounded<T>(v.z * scale) * w.z, rounded<T>(v.w * scale) * w.w));
      }
    }
    return;
  }
  if (delta != nullptr) {
    const T* d = delta + base;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float v = s[i] + to_float(d[i]);
      s[i] = v;
      acc += v * v;
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float v = s[i];
      acc += v * v;
    }
  }
  const float total = block_sum(acc, scratch);
  const float scale = rsqrtf(total / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = from_float<T>(rounded<T>(s[i] * scale) * weight[i]);
}

// ---- RMSNorm of rows [tokens, heads, width]: one wave per (token, head); input may be a strided view -------
template <typename T>
__global__ void rmsnorm_rows_kernel(const T* __restrict__ x, long token_stride, const float* __restrict__ weight,
                                    float eps, T* __restrict__ out, long rows, int heads, int width) {
  const long row = static_cast<long>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (row >= rows) return;
  const int lane = threadIdx.x & (kWave - 1);
  const T* src = x + (row / heads) * token_stride + (row % heads) * static_cast<long>(width);
  T* dst = out + row * width;
  float acc = 0.f;
  for (int i = lane; i < width; i += kWave) {
    const float v = to_float(src[i]);
    acc += v * v;
  }
  const float scale = rsqrtf(wave_sum(acc) / static_cast<float>(width) + eps);
  for (int i = lane; i < width; i += kWave) dst[i] = from_float<T>(rounded<T>(to_float(src[i]) * scale) * weight[i]);
}

template <typename T>
__global__ void copy_rows_kernel(const T* __restrict__ x, long token_stride, T* __restrict__ out, long rows,
                                 int heads, int width) {
  const long row = static_cast<long>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (row >= rows) return;
  const T* src = x + (row / heads) * token_stride + (row % heads) * static_cast<long>(width);
  for (int i = threadIdx.x & (kWave - 1); i < width; i += kWave) out[row * width + i] = src[i];
}

// ---- out[m, :] = stream[rows[m], :] (+ pending[rows[m], :]) in float32 ---------------------------------------
template <typename T>
__global__ void gather_rows_kernel(const float* __restrict__ stream, const T* __restrict__ pending,
                                   const int* __restrict__ rows, float* __restrict__ out, int hidden, int tokens) {
  const int row = rows[blockIdx.x];
  float* dst = out + static_cast<size_t>(blockIdx.x) * hidden;
  if (row < 0 || row >= tokens) {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  const size_t base = static_cast<size_t>(row) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    dst[i] = stream[base + i] + (pending != nullptr ? to_float(pending[base + i]) : 0.f);
}

// ---- SwiGLU: out[n, i] = silu(gate_up[n, i]) * gate_up[n, inter + i] ----------------------------------------
// A thread handles 8 consecutive bfloat16 outputs or 4 float32 ones (16-byte accesses) when `inter` allows.
template <typename T> long swiglu_threads(long tokens, int inter) {
  if (std::is_same<T, bf16_t>::value && (inter & 7) == 0) return tokens * (inter / 8);
  return (inter & 3) == 0 ? tokens * (inter / 4) : tokens * inter;
}
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, long tokens, int inter) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if constexpr (std::is_same<T, bf16_t>::value) {
    if ((inter & 7) == 0) {   // 16-byte accesses; the stacked product is read once and never again
      const int octets = inter / 8;
      if (index >= tokens * octets) return;
      const long n = index / octets;
      const int i = static_cast<int>(index % octets) * 8;
      typedef __attribute__((ext_vector_type(4))) unsigned int words4;
      const words4 gw = __builtin_nontemporal_load(reinterpret_cast<const words4*>(gate_up + n * 2 * inter + i));
      const words4 uw = __builtin_nontemporal_load(reinterpret_cast<const words4*>(gate_up + n * 2 * inter + inter + i));
      words4 pw;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
        pw[j] = bf16_pair(g0 / (1.f + expf(-g0)) * u0, g1 / (1.f + expf(-g1)) * u1);
      }
      *reinterpret_cast<words4*>(out + n * inter + i) = pw;
      return;
    }
  }
  if ((inter & 3) == 0) {
    const int quads = inter / 4;
    if (index >= tokens * quads) return;
    const long n = index / quads;
    const int i = static_cast<int>(index % quads) * 4;
    const float4 g = load4<T>(gate_up + n * 2 * inter + i), u = load4<T>(gate_up + n * 2 * inter + inter + i);
    store4<T>(out + n * inter + i, make_float4(g.x / (1.f + expf(-g.x)) * u.x, g.y / (1.f + expf(-g.y)) * u.y,
                                               g.z / (1.f + expf(-g.z)) * u.z, g.w / (1.f + expf(-g.w)) * u.w));
    return;
  }
  if (index >= tokens * inter) return;
  const long n = index / inter;
  const int i = static_cast<int>(index % inter);
  const float g = to_float(gate_up[n * 2 * inter + i]);
  const float u = to_float(gate_up[n * 2 * inter + inter + i]);
  out[index] = from_float<T>(g / (1.f + expf(-g)) * u);
}

// ---- rotary table: table[p, j] = (cos, sin)(p * inv_freq[j]) in float32 --------------------------------------
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, float* __restrict__ table, int positions,
                                  int half) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= static_cast<long>(positions) * half) return;
  const float angle = static_cast<float>(index / half) * inv_freq[index % half];
  float s, c;
  sincosf(angle, &s, &c);
  table[2 * index] = c;
  table[2 * index + 1] = s;
}

// ---- rotation in place of x [tokens, heads, dim]: pairs (j, j + dim/2) ----------------------------------------
template <typename T>
__global__ void rope_kernel(T* __restrict__ x, const int* __restrict__ positions, const float* __restrict__ table,
                            long tokens, int heads, int dim, int table_positions) {
  const int half = dim / 2;
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= tokens * heads * half) return;
  const int j = static_cast<int>(index % half);
  const long row = index / half;  // token * heads + head
  const int pos = positions[row / heads];
  T* p = x + row * dim;
  if (pos < 0 || pos >= table_positions) {
    p[j] = from_float<T>(__uint_as_float(0x7fc00000u));
    p[j + half] = from_float<T>(__uint_as_float(0x7fc00000u));
    return;
  }
  const float c = table[(static_cast<long>(pos) * half + j) * 2], s = table[(static_cast<long>(pos) * half + j) * 2 + 1];
  const float lo = to_float(p[j]), hi = to_float(p[j + half]);
  p[j] = from_float<T>(lo * c - hi * s);
  p[j + half] = from_float<T>(hi * c + lo * s);
}

// ---- cache write; slot = page * page_size + offset -----------------------------------------------------------
// Key pages are [num_pages, kv_heads, page_size, dim] (a key's dims are contiguous: the score product runs over
// them); value pages are [num_pages, kv_heads, dim, page_size] (a dim's keys are contiguous: the weighted sum runs
// over keys), so that both reach the matrix cores without a transposition.
template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride,
                                const int* __restrict__ slot_map, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                long tokens, int kv_heads, int dim, int page_size, long num_slots) {
  const long row = static_cast<long>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (row >= tokens * kv_heads) return;
  const long n = row / kv_heads;
  const int h = static_cast<int>(row % kv_heads);
  const long slot = slot_map[n];
  if (slot < 0 || slot >= num_slots) return;  // host checks the map; never write outside the pool
  const long page = slot / page_size, offset = slot % page_size;
  const long k_at = ((page * kv_heads + h) * page_size + offset) * dim;
  const long v_at = (page * kv_heads + h) * dim * page_size + offset;
  const T* ks = k + n * k_stride + static_cast<long>(h) * dim;
  const T* vs = v + n * v_stride + static_cast<long>(h) * dim;
  for (int i = threadIdx.x & (kWave - 1); i < dim; i += kWave) {
    k_pages[k_at + i] = ks[i];
    v_pages[v_at + static_cast<long>(i) * page_size] = vs[i];
  }
}

// ---- fused: per-head RMSNorm of q and k, rotation of q and k, q out, k and v into the token's cache slot -------
// A head of a qkv row belongs to dim / 16 neighbouring lanes; a lane owns 8 consecutive rotation pairs
// (j, j + dim/2), j = 8 * part .. + 7, read and written as two pieces of 8 elements (16 bytes of bfloat16), so the
// rotation needs no exchange between lanes and a wave works on 64 / (dim / 16) heads of one token at once.  The sum
// of squares of a head is formed in the same order in every lane of the head.  Any step can be switched off:
// q_weight/k_weight null (no norm), table null (no rotation), slot_map null (no cache write).
template <typename T> __device__ __forceinline__ void load8(const T* p, float (&v)[8]);
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <> __device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float (&v)[8]) {
  const uint4 u = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
// The same in two steps - the registers as they come from memory, and their eight values -, for code that wants all
// its loads on their way before the first of them is looked at.
template <typename T> struct Raw8;
template <> struct Raw8<float> { float4 a, b; };
template <> struct Raw8<bf16_t> { uint4 u; };
__device__ __forceinline__ Raw8<float> fetch8(const float* p) {
  return Raw8<float>{*reinterpret_cast<const float4*>(p), *reinterpret_cast<const float4*>(p + 4)};
}
__device__ __forceinline__ Raw8<bf16_t> fetch8(const bf16_t* p) { return Raw8<bf16_t>{*reinterpret_cast<const uint4*>(p)}; }
__device__ __forceinline__ void unpack8(const Raw8<float>& r, float (&v)[8]) {
  v[0] = r.a.x; v[1] = r.a.y; v[2] = r.a.z; v[3] = r.a.w; v[4] = r.b.x; v[5] = r.b.y; v[6] = r.b.z; v[7] = r.b.w;
}
__device__ __forceinline__ void unpack8(const Raw8<bf16_t>& r, float (&v)[8]) {
  const uint32_t w[4] = {r.u.x, r.u.y, r.u.z, r.u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
template <typename T> __device__ __forceinline__ void store8(T* p, const float (&v)[8]);
template <> __device__ __forceinline__ void store8<float>(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <> __device__ __forceinline__ void store8<bf16_t>(bf16_t* p, const float (&v)[8]) {
  uint4 u;
  u.x = bf16_pair(v[0], v[1]);
  u.y = bf16_pair(v[2], v[3]);
  u.z = bf16_pair(v[4], v[5]);
  u.w = bf16_pair(v[6], v[7]);
  *reinterpret_cast<uint4*>(p) = u;
}

// Values of eight consecutive rows of the step and one kv head, written by one wave.  A value page lies
// [dim, page_size]: a token's value is `dim` elements that are page_size apart, and written token by token that is
// `dim` two-byte stores per head.  Here a lane takes two dims of eight tokens (eight 4-byte reads, each token's row
// read by the wave as one piece); when the eight tokens' slots follow each other from a multiple of eight inside one
// page - portions of prompts mostly do - it writes each dim's eight tokens as ONE 16-byte store.  Otherwise, and for
// storage that is not 2 bytes wide, element by element.
template <typename T>
__device__ __forceinline__ void write_values_by_eights(const T* __restrict__ qkv, const int* __restrict__ slot_map,
                                                       T* __restrict__ v_pages, long tokens, int q_heads, int kv_heads,
                                                       int dim, int page_size, long num_slots, long item, int lane) {
  const long groups = (tokens + 7) / 8;
  if (item >= groups * kv_heads) return;
  const long n0 = (item / kv_heads) * 8;
  const int h = static_cast<int>(item % kv_heads);
  const long row = static_cast<long>(q_heads + 2 * kv_heads) * dim;
  long slot[8];
  bool together = (page_size & 7) == 0 && sizeof(T) == 2;
#pragma unroll
  for (int t = 0; t < 8; ++t) slot[t] = slot_map[min(n0 + t, tokens - 1)];   // (all eight asked for at once)
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    if (n0 + t >= tokens || slot[t] < 0 || slot[t] >= num_slots) slot[t] = -1;  // host checks the map; never write outside the pool
    together = together && slot[t] >= 0 && slot[t] == slot[0] + t;
  }
  together = together && (slot[0] & 7) == 0;
  const T* src = qkv + static_cast<long>(q_heads + kv_heads + h) * dim;
  for (int d = 2 * lane; d < dim; d += 2 * kWave) {
    // All eight tokens' loads go out together, whatever their slots (a token beyond the last reads the last one's
    // row; what has no slot is set to zero afterwards): behind a test each, they are waited for one by one - eight
    // trips to memory instead of one.
    T pair[8][2];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const T* from = src + min(n0 + t, tokens - 1) * row + d;
      pair[t][0] = from[0];
      pair[t][1] = from[1];
    }
#pragma unroll
    for (int t = 0; t < 8; ++t)
      if (slot[t] < 0) pair[t][0] = pair[t][1] = T{};
    if constexpr (sizeof(T) == 2) {
      if (together) {
        const long page = slot[0] / page_size, offset = slot[0] % page_size;
        T* dst = v_pages + ((page * kv_heads + h) * dim + d) * page_size + offset;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          T line[8];
#pragma unroll
          for (int t = 0; t < 8; ++t) line[t] = pair[t][e];
          *reinterpret_cast<uint4*>(dst + static_cast<long>(e) * page_size) = *reinterpret_cast<const uint4*>(line);
        }
        continue;
      }
    }
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      if (slot[t] < 0) continue;
      const long page = slot[t] / page_size, offset = slot[t] % page_size;
      T* dst = v_pages + ((page * kv_heads + h) * dim + d) * page_size + offset;
      dst[0] = pair[t][0];
      dst[page_size] = pair[t][1];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_write_kernel(
    const T* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ table, int table_positions, const int* __restrict__ positions,
    const int* __restrict__ slot_map, T* __restrict__ k_pages, T* __restrict__ v_pages, T* __restrict__ q_out,
    long tokens, int q_heads, int kv_heads, int dim, int page_size, long num_slots, unsigned value_blocks) {
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  // value_blocks: 0xffffffff - values are written like keys, by the lanes of their heads; else the first so many
  // blocks write them, eight tokens at a time (see above; they take longest, so they start first)
  const bool values_apart = value_blocks != 0xffffffffu;
  if (values_apart && blockIdx.x < value_blocks) {
    write_values_by_eights<T>(qkv, slot_map, v_pages, tokens, q_heads, kv_heads, dim, page_size, num_slots,
                              static_cast<long>(blockIdx.x) * waves + wave, lane);
    return;
  }
  const unsigned block = values_apart ? blockIdx.x - value_blocks : blockIdx.x;
  const int lanes_per_head = dim / 16, heads_per_wave = kWave / lanes_per_head;
  // with blocks of their own for the values, the heads of this part are the query and key heads alone
  const int row_heads = q_heads + 2 * kv_heads;
  const int heads = values_apart ? q_heads + kv_heads : row_heads;
  const int groups = (heads + heads_per_wave - 1) / heads_per_wave;
  const long item = static_cast<long>(block) * waves + wave;
  if (item >= tokens * groups) return;
  const long n = item / groups;
  const int sub = lane / lanes_per_head, part = lane % lanes_per_head;
  const int h = static_cast<int>(item % groups) * heads_per_wave + sub;
  const bool active = sub < heads_per_wave && h < heads;
  const bool is_q = h < q_heads, is_v = h >= q_heads + kv_heads;
  const int half = dim / 2, j0 = part * 8;
  const float nan = __uint_as_float(0x7fc00000u);
  const bool normed = q_weight != nullptr;

  // Every load goes out before anything waits, and none stands behind a test of what a lane is: a lane without a
  // head reads the row's last head, a position without angles the table's first row, and what must not count is
  // dropped afterwards.  (Behind tests the compiler waits for each group of loads where the paths meet again: a
  // trip to memory for the row, one for the position, one for the angles, one for the weights.)  The tests left are
  // those of the launch - no table, no norm, no cache -, the same for every lane.
  const int h_read = min(h, row_heads - 1);
  const T* src = qkv + (n * row_heads + h_read) * dim;
  const Raw8<T> raw_lo = fetch8(src + j0), raw_hi = fetch8(src + half + j0);
  long slot = (slot_map != nullptr ? slot_map : positions)[n];   // (no cache: any integer of the token, dropped below)
  const int pos = positions[n];
  Raw8<float> raw_w_lo{}, raw_w_hi{};
  if (normed) {
    const float* w = is_q ? q_weight : k_weight;
    raw_w_lo = fetch8(w + j0);
    raw_w_hi = fetch8(w + half + j0);
  }
  float4 angles[4] = {};
  const bool known = pos >= 0 && pos < table_positions;
  if (table != nullptr) {
    const float* at = table + (static_cast<long>(known ? pos : 0) * half + j0) * 2;  // (cos, sin) pairs of 8 consecutive j
#pragma unroll
    for (int q = 0; q < 4; ++q) angles[q] = *reinterpret_cast<const float4*>(at + 4 * q);
  }
  __builtin_amdgcn_sched_barrier(0);

  if (slot_map == nullptr || slot < 0 || slot >= num_slots) slot = -1;  // host checks the map; never write outside the pool
  const long page = slot >= 0 ? slot / page_size : 0, offset = slot >= 0 ? slot % page_size : 0;
  const bool works = active && (is_q || slot >= 0);  // keys and values of a token without a slot go nowhere
  const bool turns = works && !is_v;  // a query or key head: normed and rotated
  float lo[8], hi[8], cs[8], sn[8], w_lo[8], w_hi[8];
  unpack8(raw_lo, lo);
  unpack8(raw_hi, hi);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if (!works) lo[e] = hi[e] = 0.f;
    sn[e] = 0.f;
    cs[e] = w_lo[e] = w_hi[e] = 1.f;
  }
  if (table != nullptr) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      cs[2 * q] = known ? angles[q].x : nan;
      sn[2 * q] = known ? angles[q].y : nan;
      cs[2 * q + 1] = known ? angles[q].z : nan;
      sn[2 * q + 1] = known ? angles[q].w : nan;
    }
  }
  if (normed) {
    unpack8(raw_w_lo, w_lo);
    unpack8(raw_w_hi, w_hi);
  }
  if (works && is_v) {  // value: copied as it is, into the [dim, page_size] layout
    T* dst = v_pages + (page * kv_heads + (h - q_heads - kv_heads)) * dim * page_size + offset;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      dst[static_cast<long>(j0 + e) * page_size] = from_float<T>(lo[e]);
      dst[static_cast<long>(half + j0 + e) * page_size] = from_float<T>(hi[e]);
    }
  }
  // the head's sum of squares; every lane of the head ends with the same bits (a butterfly adds the same two numbers
  // on both sides; otherwise the parts are added in the same order by every lane)
  float total = 0.f;
  if (normed) {
    float own = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) own += lo[e] * lo[e] + hi[e] * hi[e];
    if ((lanes_per_head & (lanes_per_head - 1)) == 0) {
      total = own;
      for (int step = 1; step < lanes_per_head; step <<= 1) total += __shfl_xor(total, step, kWave);
    } else {
      for (int p = 0; p < lanes_per_head; ++p) total += __shfl(own, sub * lanes_per_head + p, kWave);
    }
  }
  if (!turns) return;
  if (normed) {  // normalise, round to the activation type, times the weight, round again
    const float scale = rsqrtf(total / static_cast<float>(dim) + eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      lo[e] = rounded<T>(rounded<T>(lo[e] * scale) * w_lo[e]);
      hi[e] = rounded<T>(rounded<T>(hi[e] * scale) * w_hi[e]);
    }
  }
  float out_lo[8], out_hi[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    out_lo[e] = lo[e] * cs[e] - hi[e] * sn[e];
    out_hi[e] = hi[e] * cs[e] + lo[e] * sn[e];
  }
  T* dst = is_q ? q_out + (n * q_heads + h) * dim
                : k_pages + ((page * kv_heads + (h - q_heads)) * page_size + offset) * dim;
  store8<T>(dst + j0, out_lo);
  store8<T>(dst + half + j0, out_hi);
}

inline unsigned blocks_for(long items, int per_block) { return static_cast<unsigned>((items + per_block - 1) / per_block); }

// What a kernel that only reads can draw from memory: every wave walks its own contiguous span in pieces of 1 KB, eight
// loads in flight, marked as read-once - the access pattern of the decode products' weights without any of their work.
// The words are folded with xor, a word per block, so that the reads cannot be dropped and a test can check them.
typedef unsigned int probe_uintx4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void read_probe_kernel(const probe_uintx4* __restrict__ data, long pieces, unsigned int* out) {
  constexpr int U = 8;
  __shared__ unsigned int folded[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long waves = static_cast<long>(gridDim.x) * 4, tiles = pieces / 64;   // a tile: 64 pieces of 16 bytes
  const long mine = static_cast<long>(blockIdx.x) * 4 + wave;
  const long t0 = tiles * mine / waves, t1 = tiles * (mine + 1) / waves;
  unsigned int word = 0;
  for (long t = t0; t < t1; t += U) {
    probe_uintx4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(data + min(t + u, t1 - 1) * 64 + lane);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (t + u < t1) word ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (mine == waves - 1)   // the pieces beyond the last whole tile
    for (long p = tiles * 64 + lane; p < pieces; p += 64) word ^= data[p].x ^ data[p].y ^ data[p].z ^ data[p].w;
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) word ^= __shfl_xor(word, offset, kWave);
  if (lane == 0) folded[wave] = word;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = folded[0] ^ folded[1] ^ folded[2] ^ folded[3];
}

}  // namespace

extern "C" {

// `seq_of_token`, `seq_slots`, `slot_words` (all three or none): where an id of -1 finds the token chosen last for its
// request.  Without them -1 is an id outside the table like any other.
int akv_embed(const int* ids, const void* table, int table_dtype, float* out, int tokens, int hidden, int vocab,
              const int* seq_of_token, const int* seq_slots, const int* slot_words, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (slot_words != nullptr && (seq_of_token == nullptr || seq_slots == nullptr)) return -2;
  AKV_DISPATCH(table_dtype, T,
               embed_kernel<T><<<tokens, 256, 0, stream>>>(ids, static_cast<const T*>(table), out, hidden, vocab,
                                                           seq_of_token, seq_slots, slot_words));
  return AKV_LAUNCH_STATUS();
}

// state[patches[2 i]] = patches[2 i + 1] for i < min(count[0], capacity), and the slots' lengths:
// state[seq_slots[r] * 8] = seq_lens[r] for r < seqs.  `count` lives on the device, so a recorded step applies
// however many changes the replayed step brings, up to the capacity it was recorded with.
int akv_step_prologue(int* state, long state_size, const int* patches, const int* count, int capacity,
                      const int* seq_slots, const int* seq_lens, int seqs, hipStream_t stream) {
  const int threads = capacity > seqs ? capacity : seqs;
  if (threads <= 0) return 0;
  if (state_size <= 0 || capacity < 0 || seqs < 0) return -2;
  step_prologue_kernel<<<(threads + 255) / 256, 256, 0, stream>>>(state, state_size, patches, count, capacity, seq_slots,
                                                                  seq_lens, seqs);
  return AKV_LAUNCH_STATUS();
}

int akv_add_rmsnorm(float* stream_buf, const void* delta, const float* weight, float eps, void* out, int dtype,
                    int tokens, int hidden, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 4096) {
    AKV_DISPATCH(dtype, T, (add_rmsnorm_kernel<T, 4><<<tokens, 256, 0, stream>>>(
                               stream_buf, static_cast<const T*>(delta), weight, eps, static_cast<T*>(out), hidden)));
  } else if (hidden <= 8192) {
    AKV_DISPATCH(dtype, T, (add_rmsnorm_kernel<T, 8><<<tokens, 256, 0, stream>>>(
                               stream_buf, static_cast<const T*>(delta), weight, eps, static_cast<T*>(out), hidden)));
  } else {
    AKV_DISPATCH(dtype, T, (add_rmsnorm_kernel<T, 16><<<tokens, 256, 0, stream>>>(
                               stream_buf, static_cast<const T*>(delta), weight, eps, static_cast<T*>(out), hidden)));
  }
  return AKV_LAUNCH_STATUS();
}

int akv_rmsnorm_rows(const void* x, long token_stride, const float* weight, float eps, void* out, int dtype,
                     long tokens, int heads, int width, hipStream_t stream) {
  const long rows = tokens * heads;
  if (rows <= 0) return 0;
  AKV_DISPATCH(dtype, T,
               rmsnorm_rows_kernel<T><<<blocks_for(rows, 4), 256, 0, stream>>>(
                   static_cast<const T*>(x), token_stride, weight, eps, static_cast<T*>(out), rows, heads, width));
  return AKV_LAUNCH_STATUS();
}

int akv_copy_rows(const void* x, long token_stride, void* out, int dtype, long tokens, int heads, int width,
                  hipStream_t stream) {
  const long rows = tokens * heads;
  if (rows <= 0) return 0;
  AKV_DISPATCH(dtype, T,
               copy_rows_kernel<T><<<blocks_for(rows, 4), 256, 0, stream>>>(static_cast<const T*>(x), token_stride,
                                                                            static_cast<T*>(out), rows, heads, width));
  return AKV_LAUNCH_STATUS();
}

int akv_gather_rows(const float* stream_buf, const void* pending, int dtype, const int* rows, float* out, int wanted,
                    int hidden, int tokens, hipStream_t stream) {
  if (wanted <= 0) return 0;
  AKV_DISPATCH(dtype, T,
               gather_rows_kernel<T><<<wanted, 256, 0, stream>>>(stream_buf, static_cast<const T*>(pending), rows, out,
                                                                 hidden, tokens));
  return AKV_LAUNCH_STATUS();
}

int akv_read_probe(const void* data, long bytes, unsigned int* out, int blocks, hipStream_t stream) {
  if (bytes <= 0 || (bytes & 15) != 0 || blocks <= 0) return -2;
  read_probe_kernel<<<blocks, 256, 0, stream>>>(static_cast<const probe_uintx4*>(data), bytes / 16, out);
  return AKV_LAUNCH_STATUS();
}

int akv_swiglu(const void* gate_up, void* out, int dtype, long tokens, int inter, hipStream_t stream) {
  if (tokens <= 0) return 0;
  AKV_DISPATCH(dtype, T,
               swiglu_kernel<T><<<blocks_for(swiglu_threads<T>(tokens, inter), 256), 256, 0, stream>>>(
                   static_cast<const T*>(gate_up), static_cast<T*>(out), tokens, inter));
  return AKV_LAUNCH_STATUS();
}

int akv_rope_table(const float* inv_freq, float* table, int positions, int half, hipStream_t stream) {
  rope_table_kernel<<<blocks_for(static_cast<long>(positions) * half, 256), 256, 0, stream>>>(inv_freq, table,
                                                                                              positions, half);
  return AKV_LAUNCH_STATUS();
}

int akv_rope(void* x, int dtype, const int* positions, const float* table, long tokens, int heads, int dim,
             int table_positions, hipStream_t stream) {
  if (tokens <= 0) return 0;
  AKV_DISPATCH(dtype, T,
               rope_kernel<T><<<blocks_for(tokens * heads * (dim / 2), 256), 256, 0, stream>>>(
                   static_cast<T*>(x), positions, table, tokens, heads, dim, table_positions));
  return AKV_LAUNCH_STATUS();
}

int akv_kv_write(const void* k, long k_stride, const void* v, long v_stride, const int* slot_map, void* k_pages,
                 void* v_pages, int dtype, long tokens, int kv_heads, int dim, int page_size, long num_pages,
                 hipStream_t stream) {
  if (tokens <= 0) return 0;
  AKV_DISPATCH(dtype, T,
               kv_write_kernel<T><<<blocks_for(tokens * kv_heads, 4), 256, 0, stream>>>(
                   static_cast<const T*>(k), k_stride, static_cast<const T*>(v), v_stride, slot_map,
                   static_cast<T*>(k_pages), static_cast<T*>(v_pages), tokens, kv_heads, dim, page_size,
                   num_pages * page_size));
  return AKV_LAUNCH_STATUS();
}

int akv_qk_norm_rope_write(const void* qkv, const float* q_weight, const float* k_weight, float eps,
                           const float* table, int table_positions, const int* positions, const int* slot_map,
                           void* k_pages, void* v_pages, void* q_out, int dtype, long tokens, int q_heads,
                           int kv_heads, int dim, int page_size, long num_pages, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if ((dim & 15) != 0 || dim > 16 * kWave) return -2;  // a head is dim / 16 lanes of one wave
  const int heads_per_wave = kWave / (dim / 16);
  // With a cache to write and several tokens, the values get blocks of their own after those of queries and keys.
  const bool values_apart = slot_map != nullptr && tokens >= 8;
  const int heads = values_apart ? q_heads + kv_heads : q_heads + 2 * kv_heads;
  const long items = tokens * ((heads + heads_per_wave - 1) / heads_per_wave);
  const long value_items = values_apart ? (tokens + 7) / 8 * kv_heads : 0;
  const unsigned first = blocks_for(items, 4), more = values_apart ? blocks_for(value_items, 4) : 0u;
  AKV_DISPATCH(dtype, T,
               qk_norm_rope_write_kernel<T><<<first + more, 256, 0, stream>>>(
                   static_cast<const T*>(qkv), q_weight, k_weight, eps, table, table_positions, positions, slot_map,
                   static_cast<T*>(k_pages), static_cast<T*>(v_pages), static_cast<T*>(q_out), tokens, q_heads,
                   kv_heads, dim, page_size, num_pages * page_size, values_apart ? more : 0xffffffffu));
  return AKV_LAUNCH_STATUS();
}

}  // extern "C"

// The slot layout the kernels were compiled with: out[0] = words per slot, out[1..7] = the indices of length, last
// token, temperature, seed low, seed high, draws, taken.  The host checks its own layout against this at load.
extern "C" int akv_slot_layout(int* out) {
  out[0] = kSlotWords, out[1] = kSlotLength, out[2] = kSlotLastToken, out[3] = kSlotTemperature, out[4] = kSlotSeedLow;
  out[5] = kSlotSeedHigh, out[6] = kSlotDraws, out[7] = kSlotTaken;
  return 0;
}
