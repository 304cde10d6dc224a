// bfloat16 attention over the paged cache on the matrix cores, for prefill portions and decode tokens alike.
// Compiled once per head size: -DAKV_HEAD_DIM=<multiple of 16, at most 256>.
//
// One wave works on a tile of 16 * NQ query columns of ONE request and ONE kv head: the columns are (token, query
// head of the group) pairs, so the heads of a group share every key and value that is loaded.  Both products are
// computed transposed, which lets keys and values go from the pages straight into MFMA A operands:
//     S^T[key][col] = K[key][:] . Q[col][:]        A = 16 keys x 32 dims of a key page   (keys lie [page_size, dim])
//     O^T[dim][col] = V^T[dim][:] . P^T[:][col]    A = 16 dims x 32 keys of a value page (values lie [dim, page_size])
// S^T comes out with a lane holding, for its column, 4 consecutive keys of each 16-key tile - which is, for a fixed
// order of the 32 key slots, exactly the B operand the second product needs; and O^T has the same column per lane
// as the softmax statistics.  Nothing is transposed, nothing goes through LDS.
// Scores, softmax (base 2, scale folded in) and the weighted sum are float32.  Keys are walked in steps of 32
// aligned to absolute positions.  With SPLIT, grid.z cuts the keys into segments whose partial results (maximum,
// sum, unnormalised output) a second kernel merges: decode has too few (request, head) pairs to fill the GPU otherwise.

#include "common.h"
#include "api.h"

#ifndef AKV_HEAD_DIM
#error "compile with -DAKV_HEAD_DIM=<head size>"
#endif

using namespace akv;

namespace {

constexpr int D = AKV_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head sizes are multiples of 16 up to 256");
constexpr int KT = (D + 31) / 32;   // 32-dim steps of the score product (the last may be half empty)
constexpr int DT = D / 16;          // 16-dim tiles of the output
constexpr int PSTRIDE = D + 4;      // floats per column of a partial result: D outputs, maximum, sum, 2 pad
constexpr float kLog2e = 1.4426950408889634f;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

__device__ __forceinline__ floatx4 mfma16(uint4 a, uint4 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

struct Args {
  const bf16_t* q;            // [tokens, q_heads * D]
  const bf16_t* k_pages;      // [pages, kv_heads, page_size, D]
  const bf16_t* v_pages;      // [pages, kv_heads, D, page_size]
  bf16_t* out;                // [tokens, q_heads * D]
  float* partial;             // SPLIT: [tile][grid.y][split][16 * NQ][PSTRIDE]
  const int* q_start;         // [requests + 1] first token row of each request
  const int* seq_lens;        // [requests] tokens held after this step
  const int* block_table;     // [requests, table_width]
  int table_width;
  int seq_first, seq_count;   // the launch covers requests seq_first .. seq_first + seq_count - 1
  int q_heads, kv_heads, group, heads_per_tile, head_groups, tokens_per_tile;
  int page_size;
  long num_pages;
  float scale_log2;           // softmax scale * log2(e)
  int window;                 // 0: none
  int seg_keys, num_splits;
};

// Which request and which of its tiles this block works on.
struct Tile {
  int request, first_row, tokens, first_pos, history;
  bool found;
};

__device__ __forceinline__ Tile find_tile(const Args& a, int slot) {
  Tile t{};
  t.found = false;
  for (int r = a.seq_first; r < a.seq_first + a.seq_count; ++r) {
    const int begin = a.q_start[r], count = a.q_start[r + 1] - begin;
    const int tiles = (count + a.tokens_per_tile - 1) / a.tokens_per_tile;
    if (slot < tiles) {
      t.request = r;
      t.first_row = begin + slot * a.tokens_per_tile;
      t.tokens = min(a.tokens_per_tile, count - slot * a.tokens_per_tile);
      t.history = a.seq_lens[r] - count;
      t.first_pos = t.history + slot * a.tokens_per_tile;
      t.found = true;
      return t;
    }
    slot -= tiles;
  }
  return t;
}

template <int NQ, bool SPLIT>
__global__ __launch_bounds__(64) void attention_mfma_kernel(const Args a) {
  const int lane = threadIdx.x, r16 = lane & 15, g = lane >> 4;
  const Tile t = find_tile(a, blockIdx.x);
  if (!t.found) return;
  const int kvh = blockIdx.y / a.head_groups, hg = blockIdx.y % a.head_groups;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  // this lane's columns: one per NQ tile
  bool col_valid[NQ];
  int col_pos[NQ], col_low[NQ];
  long col_at[NQ];  // element offset of the column's query / output row
  uint4 qreg[NQ][KT];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const int c = nq * 16 + r16;
    const int token = c / a.heads_per_tile, head_in_group = hg * a.heads_per_tile + c % a.heads_per_tile;
    col_valid[nq] = token < t.tokens && head_in_group < a.group;
    col_pos[nq] = t.first_pos + token;
    col_low[nq] = a.window > 0 ? max(0, col_pos[nq] - a.window + 1) : 0;
    col_at[nq] = (static_cast<long>(t.first_row + token) * a.q_heads + kvh * a.group + head_in_group) * D;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      const int dim = kt * 32 + g * 8;
      qreg[nq][kt] = (col_valid[nq] && dim < D) ? *reinterpret_cast<const uint4*>(a.q + col_at[nq] + dim) : zero;
    }
  }

  // keys this block looks at: every key any of its tokens may see, cut to its segment
  const int last_pos = t.first_pos + t.tokens - 1;
  int range_lo = a.window > 0 ? max(0, t.first_pos - a.window + 1) : 0;
  int range_hi = last_pos;
  if (SPLIT) {
    range_lo = max(range_lo, static_cast<int>(blockIdx.z) * a.seg_keys);
    range_hi = min(range_hi, (static_cast<int>(blockIdx.z) + 1) * a.seg_keys - 1);
  }

  float m[NQ], l[NQ];
  floatx4 o[NQ][DT];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    m[nq] = -INFINITY;
    l[nq] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[nq][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  bool poisoned = false;  // a key inside the range lies in a page that is not the request's
  const int* table = a.block_table + static_cast<long>(t.request) * a.table_width;

  for (int base = range_lo & ~31; base <= range_hi; base += 32) {
    // ---- S^T = K . Q^T for two tiles of 16 keys --------------------------------------------------------------
    floatx4 s[NQ][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int key = base + j * 16 + r16;
      const bf16_t* kp = nullptr;
      if (key >= range_lo && key <= range_hi) {
        const long page = table[key / a.page_size];
        if (page < 0 || page >= a.num_pages) poisoned = true;
        else kp = a.k_pages + ((page * a.kv_heads + kvh) * a.page_size + key % a.page_size) * D;
      }
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq) s[nq][j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const int dim = kt * 32 + g * 8;
        const uint4 kreg = (kp != nullptr && dim < D) ? *reinterpret_cast<const uint4*>(kp + dim) : zero;
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq) s[nq][j] = mfma16(kreg, qreg[nq][kt], s[nq][j]);
      }
    }
    // ---- mask, running maximum and sum per column (a column lives in the 4 lanes with the same r16) ---------------
    uint4 preg[NQ], plow[NQ];  // softmax weights as bfloat16 pairs: rounded value, and what the rounding lost
    float correction[NQ];
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      float top = -INFINITY;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = base + j * 16 + g * 4 + i;
          const bool seen = col_valid[nq] && key <= col_pos[nq] && key >= col_low[nq] && key >= range_lo && key <= range_hi;
          s[nq][j][i] = seen ? s[nq][j][i] * a.scale_log2 : -INFINITY;
          top = fmaxf(top, s[nq][j][i]);
        }
      top = fmaxf(top, __shfl_xor(top, 16, 64));
      top = fmaxf(top, __shfl_xor(top, 32, 64));
      const float m_new = fmaxf(m[nq], top);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // nothing seen yet: every weight is 0, no NaN
      correction[nq] = __builtin_amdgcn_exp2f(m[nq] - m_safe);
      float sum = 0.f;
      float p[8];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[j * 4 + i] = __builtin_amdgcn_exp2f(s[nq][j][i] - m_safe);
          sum += p[j * 4 + i];
        }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      l[nq] = l[nq] * correction[nq] + sum;
      m[nq] = m_new;
      // key slots of the second product, for lane group g: keys base + 4g .. + 3, then base + 16 + 4g .. + 3.
      // A weight enters as two bfloat16 numbers (p = high + low, 16 bits of mantissa together), so that the
      // weighted sum does not carry the 2^-9 relative error of a single bfloat16.
      uint32_t high[8], low[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        high[e] = bf16_bits(p[e]);
        low[e] = bf16_bits(p[e] - __uint_as_float(high[e] << 16));
      }
      preg[nq] = make_uint4(high[0] | (high[1] << 16), high[2] | (high[3] << 16), high[4] | (high[5] << 16), high[6] | (high[7] << 16));
      plow[nq] = make_uint4(low[0] | (low[1] << 16), low[2] | (low[3] << 16), low[4] | (low[5] << 16), low[6] | (low[7] << 16));
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[nq][dt] *= correction[nq];
    }
    // ---- O^T += V^T . P^T -------------------------------------------------------------------------------------------
    const bf16_t* vp[2];
    uint32_t keep[2][2];  // masks that zero the slots of keys beyond the range (never written, may hold anything)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int key = base + j * 16 + g * 4;
      vp[j] = nullptr;
      const int live = min(4, range_hi - key + 1);  // keys of this group of 4 that exist
      if (live > 0 && key + 3 >= range_lo) {
        const long page = table[key / a.page_size];
        if (page < 0 || page >= a.num_pages) poisoned = true;
        else vp[j] = a.v_pages + (page * a.kv_heads + kvh) * static_cast<long>(D) * a.page_size + key % a.page_size;
      }
      keep[j][0] = live >= 2 ? 0xffffffffu : (live == 1 ? 0x0000ffffu : 0u);
      keep[j][1] = live >= 4 ? 0xffffffffu : (live == 3 ? 0x0000ffffu : 0u);
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const long row = static_cast<long>(dt * 16 + r16) * a.page_size;
      uint4 vreg = zero;
      if (vp[0] != nullptr) {
        const uint2 v = *reinterpret_cast<const uint2*>(vp[0] + row);
        vreg.x = v.x & keep[0][0];
        vreg.y = v.y & keep[0][1];
      }
      if (vp[1] != nullptr) {
        const uint2 v = *reinterpret_cast<const uint2*>(vp[1] + row);
        vreg.z = v.x & keep[1][0];
        vreg.w = v.y & keep[1][1];
      }
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq) o[nq][dt] = mfma16(vreg, plow[nq], mfma16(vreg, preg[nq], o[nq][dt]));
    }
  }

  // ---- results: lane holds, per column, dims dt * 16 + 4g .. + 3 ------------------------------------------------------
  const float nan = __uint_as_float(0x7fc00000u);
  poisoned = __any(poisoned);
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    if (SPLIT) {
      const int c = nq * 16 + r16;
      float* dst = a.partial + ((((static_cast<long>(blockIdx.x) * gridDim.y + blockIdx.y) * a.num_splits + blockIdx.z) * (16 * NQ)) + c) * PSTRIDE;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<floatx4*>(dst + dt * 16 + g * 4) = o[nq][dt];
      if (g == 0) {
        dst[D] = poisoned ? nan : m[nq];
        dst[D + 1] = l[nq];
      }
    } else if (col_valid[nq]) {
      const float inv = poisoned ? nan : 1.f / l[nq];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        uint2 packed;
        packed.x = bf16_bits(o[nq][dt][0] * inv) | (static_cast<uint32_t>(bf16_bits(o[nq][dt][1] * inv)) << 16);
        packed.y = bf16_bits(o[nq][dt][2] * inv) | (static_cast<uint32_t>(bf16_bits(o[nq][dt][3] * inv)) << 16);
        *reinterpret_cast<uint2*>(a.out + col_at[nq] + dt * 16 + g * 4) = packed;
      }
    }
  }
}

// Merge of the segments' partial results: out = sum_z 2^(m_z - M) O_z / sum_z 2^(m_z - M) l_z, M = max_z m_z
// (csrc/paged_decode.cu:528-544 of the reference has the same rule in base e).  One wave per (tile, head group);
// lane = (column, quarter of the dims).
template <int NQ>
__global__ __launch_bounds__(64 * NQ) void attention_merge_kernel(const Args a) {
  const Tile t = find_tile(a, blockIdx.x);
  if (!t.found) return;
  const int kvh = blockIdx.y / a.head_groups, hg = blockIdx.y % a.head_groups;
  const int c = threadIdx.x >> 2, quarter = threadIdx.x & 3;  // 16 * NQ columns x 4 lanes
  const int token = c / a.heads_per_tile, head_in_group = hg * a.heads_per_tile + c % a.heads_per_tile;
  if (token >= t.tokens || head_in_group >= a.group) return;
  const float* src = a.partial + (((static_cast<long>(blockIdx.x) * gridDim.y + blockIdx.y) * a.num_splits) * (16 * NQ) + c) * PSTRIDE;
  const long split_stride = static_cast<long>(16 * NQ) * PSTRIDE;
  float top = -INFINITY;
  for (int z = 0; z < a.num_splits; ++z) top = fmaxf(top, src[z * split_stride + D]);  // NaN marks stay NaN below
  float denom = 0.f;
  constexpr int PER = D / 4;  // dims per lane
  float acc[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) acc[i] = 0.f;
  for (int z = 0; z < a.num_splits; ++z) {
    const float* p = src + z * split_stride;
    const float mz = p[D];
    const float w = (mz != mz) ? mz : (mz == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mz - top));
    if (w == 0.f) continue;
    denom += w * p[D + 1];
#pragma unroll
    for (int i = 0; i < PER; ++i) acc[i] += w * p[quarter * PER + i];
  }
  bf16_t* dst = a.out + (static_cast<long>(t.first_row + token) * a.q_heads + kvh * a.group + head_in_group) * D + quarter * PER;
  const float inv = 1.f / denom;
#pragma unroll
  for (int i = 0; i < PER; ++i) dst[i] = from_float<bf16_t>(acc[i] * inv);
}

template <int NQ>
int launch(const Args& a, int tiles, hipStream_t stream) {
  dim3 grid(tiles, a.kv_heads * a.head_groups, a.num_splits);
  if (a.num_splits > 1) {
    attention_mfma_kernel<NQ, true><<<grid, 64, 0, stream>>>(a);
    grid.z = 1;
    attention_merge_kernel<NQ><<<grid, 64 * NQ, 0, stream>>>(a);
  } else {
    attention_mfma_kernel<NQ, false><<<grid, 64, 0, stream>>>(a);
  }
  return AKV_LAUNCH_STATUS();
}

}  // namespace

#define AKV_CONCAT2(a, b) a##b
#define AKV_CONCAT(a, b) AKV_CONCAT2(a, b)

// Attention of requests seq_first .. seq_first + seq_count - 1 of the step.  `nq` (1, 2 or 4) sets the tile to
// 16 * nq query columns; `tiles` is the number of tiles over those requests (sum of ceil(tokens / tokens_per_tile));
// with num_splits > 1 `partial` must hold tiles * kv_heads * head_groups * num_splits * 16 * nq * (D + 4) floats.
extern "C" int AKV_CONCAT(akv_attention_mfma_d, AKV_HEAD_DIM)(
    const void* q, const void* k_pages, const void* v_pages, void* out, float* partial, const int* q_start,
    const int* seq_lens, const int* block_table, int table_width, int seq_first, int seq_count, int tiles, int nq,
    int q_heads, int kv_heads, int heads_per_tile, int head_groups, int tokens_per_tile, int page_size, long num_pages,
    float scale, int window, int seg_keys, int num_splits, hipStream_t stream) {
  if (tiles <= 0 || seq_count <= 0) return 0;
  if (page_size % 4 != 0 || q_heads % kv_heads != 0 || heads_per_tile * tokens_per_tile > 16 * nq ||
      kv_heads * head_groups > 65535 || num_splits > 65535 || num_splits < 1)
    return -2;
  Args a;
  a.q = static_cast<const bf16_t*>(q);
  a.k_pages = static_cast<const bf16_t*>(k_pages);
  a.v_pages = static_cast<const bf16_t*>(v_pages);
  a.out = static_cast<bf16_t*>(out);
  a.partial = partial;
  a.q_start = q_start;
  a.seq_lens = seq_lens;
  a.block_table = block_table;
  a.table_width = table_width;
  a.seq_first = seq_first;
  a.seq_count = seq_count;
  a.q_heads = q_heads;
  a.kv_heads = kv_heads;
  a.group = q_heads / kv_heads;
  a.heads_per_tile = heads_per_tile;
  a.head_groups = head_groups;
  a.tokens_per_tile = tokens_per_tile;
  a.page_size = page_size;
  a.num_pages = num_pages;
  a.scale_log2 = scale * kLog2e;
  a.window = window;
  a.seg_keys = seg_keys;
  a.num_splits = num_splits;
  switch (nq) {
    case 1: return launch<1>(a, tiles, stream);
    case 2: return launch<2>(a, tiles, stream);
    case 4: return launch<4>(a, tiles, stream);
    default: return -2;
  }
}
