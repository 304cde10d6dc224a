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
// aligned to absolute positions.  With SPLIT a block takes a segment of a request's keys, and a second kernel merges
// the segments' partial results (maximum, sum, unnormalised output): decode has too few (request, head) pairs to fill
// the GPU otherwise.  Single tokens' segments come from a plan made on the device from the requests' lengths (one
// segment size for all of them); prompt portions that are cut get the same number of segments each (grid.z).

#include <type_traits>

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
typedef __attribute__((ext_vector_type(2))) float floatx2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;  // 16 bytes of operand: 8 bfloat16 (plain vector
typedef __attribute__((ext_vector_type(2))) unsigned int uintx2;  // types: the compiler keeps them in registers)

__device__ __forceinline__ floatx4 mfma16(uintx4 a, uintx4 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// The maximum over the four lanes r, r + 16, r + 32 and r + 48, in all four of them: two lane swaps inside the vector
// unit (halves of the wave, then rows of 16 lanes) instead of two trips through LDS.
__device__ __forceinline__ float max_over_halves(float v) {
  const uint32_t bits = __float_as_uint(v);
  const auto swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  return fmaxf(__uint_as_float(swapped[0]), __uint_as_float(swapped[1]));
}
__device__ __forceinline__ float max_over_row_pairs(float v) {
  const uint32_t bits = __float_as_uint(v);
  const auto swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  return fmaxf(__uint_as_float(swapped[0]), __uint_as_float(swapped[1]));
}
__device__ __forceinline__ float max_over_groups(float v) { return max_over_row_pairs(max_over_halves(v)); }

// bfloat16 bits of x, rounded to nearest even with integer arithmetic - the same bits as the conversion instruction
// gives.  For the last lines of `attention_shared_kernel` only: with the instruction there the compiler allocates the
// registers of the kernel's loop differently and spills inside it (2,048 tokens: 88 -> 108 us).
__device__ __forceinline__ uint32_t bits_by_integer_rounding(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return ((u >> 16) | 0x0040u) & 0xffffu;  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

struct Args {
  const bf16_t* q;            // [tokens, q_heads * D]
  const bf16_t* k_pages;      // [pages, kv_heads, page_size, D]
  const bf16_t* v_pages;      // [pages, kv_heads, D, page_size]
  bf16_t* out;                // [tokens, q_heads * D]
  float* partial;             // SPLIT: [tile][grid.y][split][16 * NQ][PSTRIDE]
  const int* q_start;         // [requests + 1] first token row of each request
  const int* seq_lens;        // [requests] tokens held after this step
  const int* block_table;     // [requests, table_width], or, with `table_rows`, [slots, table_width]
  const int* table_rows;      // null, or [requests]: the row of the table that holds a request's pages (its slot)
  int table_width;
  int seq_first, seq_count;   // the launch covers requests seq_first .. seq_first + seq_count - 1
  int tiles;                  // tiles over those requests
  int single_tokens;          // every request of the launch brings exactly one token: tile i is request seq_first + i
  int q_heads, kv_heads, group, heads_per_tile, head_groups, tokens_per_tile;
  int page_shift;             // page_size = 1 << page_shift, at least 4
  long num_pages;
  float scale_log2;           // softmax scale * log2(e)
  int window;                 // 0: none
  int seg_keys, num_splits;
  // PLAN (single tokens, at most 64 requests per launch, instead of seg_keys / num_splits): the requests' keys were
  // cut into (request, segment) items by `akv_decode_plan`, which wrote `plan`: [0] items in all, [4 + 2 r] the items
  // before request r's and [5 + 2 r] their number, [132 + 4 i] item i's request (from seq_first), first key, token
  // position and last key.  Such a launch has grid (kv_heads * head_groups, items_grid): the items that exist come
  // first; `items_grid` is a bound the host knows.
  const int* plan;
  int items_grid;
  int units;                  // compute units of the device (block order of the shared kernel)
  // FRESH launches (single tokens whose projections have not been normed, rotated or written to the cache yet):
  const bf16_t* qkv;          // [tokens, (q_heads + 2 * kv_heads) * D]: query, key and value heads of a token in a row
  const float* q_weight;      // [D] weights of the per-head norm of queries and of keys; both null: no norm
  const float* k_weight;
  const float* rope_table;    // [table_positions, D / 2, 2] (cos, sin) per position and rotation pair; null: no rotation
  int table_positions;
  float eps;
};

// Which request and which of its tiles this block works on.
struct Tile {
  int request, first_row, tokens, first_pos;
  bool found;
};

// Tiles are numbered request by request.  The wave looks at 64 requests at a time: every lane counts the tiles of
// one request, a prefix sum over the lanes places them, and the lane whose span holds `slot` owns the answer.
__device__ __forceinline__ Tile find_tile(const Args& a, int slot, int per_tile) {
  Tile t{};
  t.found = false;
  const int lane = threadIdx.x & 63, end = a.seq_first + a.seq_count;
  if (a.single_tokens) {
    if (slot >= a.seq_count) return t;
    t.request = a.seq_first + slot;
    t.first_row = a.q_start[t.request];
    t.tokens = 1;
    t.first_pos = a.seq_lens[t.request] - 1;
    t.found = true;
    return t;
  }
  int before = 0;  // tiles of the requests already passed
  for (int r0 = a.seq_first; r0 < end; r0 += 64) {
    const int r = r0 + lane;
    int begin = 0, count = 0;
    if (r < end) {
      begin = a.q_start[r];
      count = a.q_start[r + 1] - begin;
    }
    const int tiles = (count + per_tile - 1) / per_tile;
    int upto = tiles;  // inclusive prefix sum over the wave
#pragma unroll
    for (int step = 1; step < 64; step <<= 1) {
      const int other = __shfl_up(upto, step, 64);
      if (lane >= step) upto += other;
    }
    const int total = __shfl(upto, 63, 64);
    if (slot < before + total) {
      const bool mine = slot >= before + upto - tiles && slot < before + upto;
      const int owner = __ffsll(static_cast<unsigned long long>(__ballot(mine))) - 1;
      const int local = slot - (before + __shfl(upto - tiles, owner, 64));
      const int o_begin = __shfl(begin, owner, 64), o_count = __shfl(count, owner, 64);
      t.request = r0 + owner;
      t.first_row = o_begin + local * per_tile;
      t.tokens = min(per_tile, o_count - local * per_tile);
      t.first_pos = a.seq_lens[t.request] - o_count + local * per_tile;
      t.found = true;
      return t;
    }
    before += total;
  }
  return t;
}

// A head as a lane's operand pieces (piece kt: dims kt * 32 + g * 8 .. + 7), normed over the head and rotated in place:
// x * rsqrt(mean(x^2) + eps), rounded, times the weight, rounded; then the pairs (j, j + D / 2) are turned by the
// position's angles (ampere_kv/runner.py:48-57, :88-98 of the reference).  With D a multiple of 64 the partner of
// piece kt is piece kt + KT / 2 of the same lane, and the head's sum of squares is the sum over the four lanes that
// share r16.  What it needs from memory is fetched apart (`HeadWeights`, `HeadAngles`), so that a kernel can have
// these loads and others on their way before any arithmetic waits for them.  All 64 lanes call `encode_head` together.
constexpr int KH = (KT + 1) / 2;  // pieces of the first half of a head
struct HeadWeights {
  floatx2 w[KT][4];
};
struct HeadAngles {
  floatx2 cs[KH][4], sn[KH][4];
};
__device__ __forceinline__ void fetch_weights(HeadWeights& to, const float* weight, int g) {
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float4 v = *reinterpret_cast<const float4*>(weight + kt * 32 + g * 8 + h * 4);
      to.w[kt][2 * h] = floatx2{v.x, v.y};
      to.w[kt][2 * h + 1] = floatx2{v.z, v.w};
    }
}
// `angles`: a row of the table (cos, sin per rotation pair); `poison`: the position has no row - every angle is NaN
__device__ __forceinline__ void fetch_angles(HeadAngles& to, const float* angles, bool poison, int g) {
  const float nan = __uint_as_float(0x7fc00000u);
#pragma unroll
  for (int kt = 0; kt < KT / 2; ++kt)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 v = *reinterpret_cast<const float4*>(angles + (kt * 32 + g * 8) * 2 + 4 * q);
      to.cs[kt][q] = floatx2{poison ? nan : v.x, poison ? nan : v.z};
      to.sn[kt][q] = floatx2{poison ? nan : v.y, poison ? nan : v.w};
    }
}

// rounding of two floats to bfloat16 (nearest, ties to even) in one conversion instruction, and back
__device__ __forceinline__ floatx2 rounded2(floatx2 v) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  return floatx2{__uint_as_float(bits << 16), __uint_as_float(bits & 0xffff0000u)};
}

__device__ __forceinline__ void encode_head(uintx4 (&reg)[KT], bool normed, float eps, const HeadWeights& weights,
                                            bool rotated, const HeadAngles& angles) {
  static_assert(KT % 2 == 0 || D % 64 != 0, "pieces pair up when the head size is a multiple of 64");
  floatx2 x[KT][4];
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int w = 0; w < 4; ++w) x[kt][w] = floatx2{__uint_as_float(reg[kt][w] << 16), __uint_as_float(reg[kt][w] & 0xffff0000u)};
  if (normed) {
    float squares = 0.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int w = 0; w < 4; ++w) squares += x[kt][w][0] * x[kt][w][0] + x[kt][w][1] * x[kt][w][1];
    squares += __shfl_xor(squares, 16, 64);
    squares += __shfl_xor(squares, 32, 64);
    const float scale = rsqrtf(squares / static_cast<float>(D) + eps);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int w = 0; w < 4; ++w) x[kt][w] = rounded2(rounded2(x[kt][w] * scale) * weights.w[kt][w]);
    }
  }
  if (rotated) {
#pragma unroll
    for (int kt = 0; kt < KT / 2; ++kt)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const floatx2 cs = angles.cs[kt][w], sn = angles.sn[kt][w];
        const floatx2 lo = x[kt][w], hi = x[kt + KT / 2][w];
        x[kt][w] = lo * cs - hi * sn;
        x[kt + KT / 2][w] = hi * cs + lo * sn;
      }
  }
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int w = 0; w < 4; ++w) reg[kt][w] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x[kt][w], bf16x2));
}

// Inside a step of 32 keys starting at `base`, MFMA tile j (0 or 1), row rho (0..15) is key
//     base + (rho / 4) * 8 + j * 4 + rho % 4.
// With this order the 8 score elements a lane holds (rows 4g .. 4g + 3 of both tiles) are the 8 CONSECUTIVE keys
// base + 8g .. + 7, so the value operand of lane group g is one 16-byte read of a value page row.
// PIPE: the next step's keys are fetched while this step computes (costs registers: used where they are there).
// FRESH (single tokens, D a multiple of 64): query, key and value of the token come raw from the stacked projection
// `a.qkv`.  Every block norms and rotates its own query heads in registers; the block whose keys include the token's
// own position does the same for the new key, puts it and the new value into its operands in place of what the page
// holds there, and writes both to the page for later steps.  No other block reads that slot in this launch.
// (Split launches of head sizes up to 128 are held to the registers of two waves per SIMD: decoding lives on the
// number of waves that wait for memory at the same time.)
// ONCE: no other block of the launch reads these keys and values (single tokens, one block per kv head and segment):
// the loads are marked read-once.  A bare reader with this kernel's lanes and depth draws 7.1 TB/s from 2 GB of
// pages with the mark and 6.5 TB/s without.
// (The kernel's text is a function of where a wave stands in the grid, so that another kernel can run it beside the
// prompt portions' blocks: see `attention_pair_kernel`.)
struct Where {
  int bx, by, bz, gx, gy;   // the wave's block and the grid, as blockIdx and gridDim would name them
  int lane;
};

template <int NQ, bool SPLIT, bool PIPE, bool FRESH, bool ONCE>
__device__ __forceinline__ void attention_mfma_body(const Args& a, const Where at) {
  const int lane = at.lane, r16 = lane & 15, g = lane >> 4;
  auto from_pages = [](const char* at) {
    const uintx4* p = reinterpret_cast<const uintx4*>(at);
    return ONCE ? __builtin_nontemporal_load(p) : *p;
  };
  // Without SPLIT a block works on two tiles, one after the other: tile `tiles - 1 - x` and tile `x`.  Under the
  // causal mask the late tiles of a prompt see many keys and the early ones few; a pair sees about the same number
  // as every other pair, so the blocks finish together instead of waiting for the longest.
  // (FRESH launches hold single tokens, whose tiles have nothing to balance: one tile per block, like SPLIT.)
  constexpr bool kOneTile = SPLIT || FRESH;
  for (int pass = 0; pass < (kOneTile ? 1 : 2); ++pass) {
  const int slot = kOneTile ? at.bx : (pass == 0 ? a.tiles - 1 - at.bx : at.bx);
  if (!kOneTile && pass == 1 && slot >= a.tiles - 1 - slot) break;  // the middle tile was the first pass's
  Tile t{};
  int seg_lo = 0, seg_hi = 0x7fffffff;     // SPLIT: the keys of this block's segment
  long part = 0;                           // SPLIT: index of its partial result's tile
  if (SPLIT && a.plan != nullptr) {        // item `by` of the plan: a request and a segment of its keys
    const int item = at.by;
    if (item >= a.plan[0]) return;
    const int4 record = *reinterpret_cast<const int4*>(a.plan + 132 + 4 * item);
    t.request = a.seq_first + record.x;
    t.first_row = a.q_start[a.seq_first] + record.x;   // one row per request
    t.tokens = 1;
    t.first_pos = record.z;
    t.found = true;
    seg_lo = record.y;
    seg_hi = record.w;
    part = static_cast<long>(item) * at.gx + at.bx;
  } else {
    t = find_tile(a, slot, a.tokens_per_tile);
    if (!t.found) continue;
    if (SPLIT) {
      seg_lo = at.bz * a.seg_keys;
      seg_hi = seg_lo + a.seg_keys - 1;
      part = (static_cast<long>(at.bx) * at.gy + at.by) * a.num_splits + at.bz;
    }
  }
  const int head_block = (SPLIT && a.plan != nullptr) ? at.bx : at.by;  // (kv head, group of its query heads)
  const int kvh = head_block / a.head_groups, hg = head_block % a.head_groups;
  const uintx4 zero = uintx4{0u, 0u, 0u, 0u};
  const int page_size = 1 << a.page_shift, page_mask = page_size - 1;

  // this lane's columns: one per NQ tile
  bool col_valid[NQ];
  int col_pos[NQ], col_low[NQ];
  long col_at[NQ];  // element offset of the column's query / output row
  uintx4 qreg[NQ][KT];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const int c = nq * 16 + r16;
    const int token = c / a.heads_per_tile, head_in_group = hg * a.heads_per_tile + c % a.heads_per_tile;
    col_valid[nq] = token < t.tokens && head_in_group < a.group;
    col_pos[nq] = t.first_pos + token;
    col_low[nq] = a.window > 0 ? max(0, col_pos[nq] - a.window + 1) : 0;
    col_at[nq] = (static_cast<long>(t.first_row + token) * a.q_heads + kvh * a.group + head_in_group) * D;
    // FRESH: the raw query head of the stacked row (a single token: row t.first_row)
    const bf16_t* q_from = FRESH ? a.qkv + (static_cast<long>(t.first_row) * (a.q_heads + 2 * a.kv_heads) + kvh * a.group + head_in_group) * D
                                 : a.q + col_at[nq];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      const int dim = kt * 32 + g * 8;
      qreg[nq][kt] = (col_valid[nq] && dim < D) ? *reinterpret_cast<const uintx4*>(q_from + dim) : zero;
    }
  }
  // FRESH: what the encoding of queries and the new key needs from memory is asked for here, and used only after
  // the first keys have been asked for too.
  const int new_pos = t.first_pos;
  const bool normed = FRESH && a.q_weight != nullptr, rotated = FRESH && a.rope_table != nullptr;
  HeadWeights q_weights, k_weights;
  HeadAngles head_angles;
  if constexpr (FRESH) {
    if (normed) fetch_weights(q_weights, a.q_weight, g);
    if (rotated) {
      const bool known = new_pos >= 0 && new_pos < a.table_positions;
      fetch_angles(head_angles, a.rope_table + (known ? static_cast<long>(new_pos) * D : 0L), !known, g);
    }
  }

  // keys this block looks at: every key any of its tokens may see, cut to its segment
  const int last_pos = t.first_pos + t.tokens - 1;
  int range_lo = a.window > 0 ? max(0, t.first_pos - a.window + 1) : 0;
  int range_hi = last_pos;
  if (SPLIT) {
    range_lo = max(range_lo, seg_lo);
    range_hi = min(range_hi, seg_hi);
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
  const int* table = a.block_table + static_cast<long>(a.table_rows != nullptr ? a.table_rows[t.request] : t.request) * a.table_width;
  const int key_in_step = (r16 >> 2) * 8 + (r16 & 3);  // + j * 4: this lane's key row of tile j

  // A page's byte offset is 64-bit (pools of many gigabytes); what is added inside a page fits 32 bits and is
  // prepared once per lane.
  const char* k_bytes = reinterpret_cast<const char*>(a.k_pages);
  const char* v_bytes = reinterpret_cast<const char*>(a.v_pages);
  const uint32_t page_bytes = static_cast<uint32_t>(a.kv_heads) * D * 2u << a.page_shift;  // one page, all kv heads
  const uint32_t head_bytes = static_cast<uint32_t>(kvh) * D * 2u << a.page_shift;         // this kv head inside a page
  const uint32_t k_lane = head_bytes + g * 16u;                         // + key row * D * 2 + kt * 64
  const uint32_t v_lane = head_bytes + (static_cast<uint32_t>(r16) << (a.page_shift + 1));  // + dt * 16 rows + key * 2
  const uint32_t v_tile = 32u << a.page_shift;                          // 16 value rows

  // FRESH: the block whose keys include the token's own position holds the new key as operand pieces (the same in
  // every r16) and the new value per dim row, and writes both to the token's slot (one block per kv head does).
  bool owns_new = false;
  uintx4 knew[KT];
  uint32_t vnew[DT] = {};
  if constexpr (FRESH) {
    owns_new = new_pos >= range_lo && new_pos <= range_hi;
    if (owns_new) {
      const bf16_t* row = a.qkv + static_cast<long>(t.first_row) * (a.q_heads + 2 * a.kv_heads) * D;
      const bf16_t* k_from = row + static_cast<long>(a.q_heads + kvh) * D;
      const bf16_t* v_from = row + static_cast<long>(a.q_heads + a.kv_heads + kvh) * D;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) knew[kt] = *reinterpret_cast<const uintx4*>(k_from + kt * 32 + g * 8);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vnew[dt] = v_from[dt * 16 + r16].bits;
      if (normed) fetch_weights(k_weights, a.k_weight, g);
    }
  }
  auto encode_fresh = [&]() {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      encode_head(qreg[nq], normed, a.eps, q_weights, rotated, head_angles);
      if (!col_valid[nq]) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) qreg[nq][kt] = zero;
      }
    }
    if (!owns_new) return;
    encode_head(knew, normed, a.eps, k_weights, rotated, head_angles);
    if (hg != 0) return;
    const int page = table[new_pos >> a.page_shift];
    if (page < 0 || page >= a.num_pages) {
      poisoned = true;
      return;
    }
    const size_t slot_k = static_cast<size_t>(page) * page_bytes + (k_lane + static_cast<uint32_t>(new_pos & page_mask) * (D * 2u));
    const size_t slot_v = static_cast<size_t>(page) * page_bytes + (v_lane + static_cast<uint32_t>(new_pos & page_mask) * 2u);
    char* k_out = const_cast<char*>(k_bytes);  // the pages are this launch's to write at this one slot
    char* v_out = const_cast<char*>(v_bytes);
    if (r16 == 0) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<uintx4*>(k_out + slot_k + kt * 64u) = knew[kt];
    }
    if (g == 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<uint16_t*>(v_out + slot_v + dt * v_tile) = static_cast<uint16_t>(vnew[dt]);
    }
  };

  // Keys of the step at `base` into A operands.  CHECK: the step may reach outside [range_lo, range_hi]; rows outside
  // are zero and never looked up.
  auto load_keys = [&](int base, uintx4 (&dst)[2][KT], auto check) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int key = base + key_in_step + j * 4;
      const bool wanted = !decltype(check)::value || (key >= range_lo && key <= range_hi);
      int page = 0;
      if (wanted) {
        page = table[key >> a.page_shift];
        if (page < 0 || page >= a.num_pages) {
          poisoned = true;
          page = 0;
        }
      }
      const size_t at = static_cast<size_t>(page) * page_bytes + (k_lane + static_cast<uint32_t>(key & page_mask) * (D * 2u));
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const bool inside = (D % 32 == 0) || kt * 32 + g * 8 < D;
        dst[j][kt] = (wanted && inside) ? from_pages(k_bytes + at + kt * 64u) : zero;
      }
    }
  };
  // Values of the step at `base` into A operands: lane (dim row r16 of tile dt, keys base + 8g .. + 7).  CHECK: slots
  // of keys beyond the range are zeroed (they were never written and may hold anything, NaN included).
  auto load_values = [&](int base, uintx4 (&dst)[DT], auto check) {
    const int key = base + g * 8;
    if (!decltype(check)::value && page_size >= 8) {
      int page = table[key >> a.page_shift];
      if (page < 0 || page >= a.num_pages) {
        poisoned = true;
        page = 0;
      }
      const size_t at = static_cast<size_t>(page) * page_bytes + (v_lane + static_cast<uint32_t>(key & page_mask) * 2u);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) dst[dt] = from_pages(v_bytes + at + dt * v_tile);
      return;
    }
    const int live = min(8, range_hi - key + 1);
    bool have[2] = {false, false};
    size_t at[2] = {0u, 0u};
    if (live > 0 && key + 7 >= range_lo) {
      // pages of 8 and more hold the 8 keys together; pages of 4 hold them in two pages
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int first = key + half * 4;
        if (half == 1 && (page_size >= 8 || live <= 4)) break;
        if (half == 0 && page_size < 8 && key + 3 < range_lo) continue;
        const int page = table[first >> a.page_shift];
        if (page < 0 || page >= a.num_pages) poisoned = true;
        else {
          have[half] = true;
          at[half] = static_cast<size_t>(page) * page_bytes + (v_lane + static_cast<uint32_t>(first & page_mask) * 2u);
        }
      }
    }
    uint32_t keep[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) keep[w] = live >= 2 * w + 2 ? 0xffffffffu : (live == 2 * w + 1 ? 0x0000ffffu : 0u);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uintx4 v = zero;
      if (page_size >= 8) {
        if (have[0]) v = from_pages(v_bytes + at[0] + dt * v_tile);
      } else {
        if (have[0]) {
          const uintx2 h = *reinterpret_cast<const uintx2*>(v_bytes + at[0] + dt * v_tile);
          v.x = h.x;
          v.y = h.y;
        }
        if (have[1]) {
          const uintx2 h = *reinterpret_cast<const uintx2*>(v_bytes + at[1] + dt * v_tile);
          v.z = h.x;
          v.w = h.y;
        }
      }
      dst[dt] = uintx4{v.x & keep[0], v.y & keep[1], v.z & keep[2], v.w & keep[3]};
    }
  };

  uintx4 kreg[2][KT], knext[PIPE ? 2 : 1][PIPE ? KT : 1], vreg[DT];
  const std::true_type checked{};
  const std::false_type unchecked{};
  auto inside = [&](int base) { return base >= range_lo && base + 31 <= range_hi; };

  // One step of 32 keys.  MASK: some column does not see the whole step (diagonal, window, segment edge).
  auto step = [&](int base, const uintx4 (&kreg)[2][KT], auto mask) {
    // ---- S^T = K . Q^T for two tiles of 16 keys --------------------------------------------------------------
    floatx4 s[NQ][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq) s[nq][j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq) s[nq][j] = mfma16(kreg[j][kt], qreg[nq][kt], s[nq][j]);
    }
    // ---- running maximum and sum per column (a column lives in the 4 lanes with the same r16) ---------------------
    uintx4 preg[NQ], plow[NQ];  // softmax weights as bfloat16 pairs: rounded value, and what the rounding lost
    float correction[NQ];
    bool rescale = false;
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      if (decltype(mask)::value) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = base + g * 8 + j * 4 + i;
            const bool seen = col_valid[nq] && key <= col_pos[nq] && key >= col_low[nq] && key >= range_lo && key <= range_hi;
            if (!seen) s[nq][j][i] = -INFINITY;
          }
      }
      float top = fmaxf(fmaxf(fmaxf(s[nq][0][0], s[nq][0][1]), fmaxf(s[nq][0][2], s[nq][0][3])),
                        fmaxf(fmaxf(s[nq][1][0], s[nq][1][1]), fmaxf(s[nq][1][2], s[nq][1][3])));
      top = max_over_groups(top);
      const float m_new = fmaxf(m[nq], top * a.scale_log2);   // the scale is positive: max commutes with it
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // nothing seen yet: every weight is 0, no NaN
      correction[nq] = __builtin_amdgcn_exp2f(m[nq] - m_safe);
      rescale = rescale || correction[nq] != 1.f;
      floatx2 p[4];
      float sum = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        p[e][0] = __builtin_amdgcn_exp2f(fmaf(s[nq][e >> 1][(e & 1) * 2], a.scale_log2, -m_safe));
        p[e][1] = __builtin_amdgcn_exp2f(fmaf(s[nq][e >> 1][(e & 1) * 2 + 1], a.scale_log2, -m_safe));
        sum += p[e][0] + p[e][1];
      }
      l[nq] = l[nq] * correction[nq] + sum;  // this lane's own 8 keys; the 4 lanes of a column are added at the end
      m[nq] = m_new;
      // A weight enters the second product as two bfloat16 numbers (p = high + low, 16 bits of mantissa together),
      // so that the weighted sum does not carry the 2^-9 relative error of a single bfloat16.
      uint32_t high[4], low[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        high[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(p[e], bf16x2));
        const floatx2 rest = {p[e][0] - __uint_as_float(high[e] << 16), p[e][1] - __uint_as_float(high[e] & 0xffff0000u)};
        low[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2));
      }
      preg[nq] = uintx4{high[0], high[1], high[2], high[3]};
      plow[nq] = uintx4{low[0], low[1], low[2], low[3]};
    }
    if (__any(rescale)) {  // the maxima rarely move after the first steps
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[nq][dt] *= correction[nq];
    }
    // ---- O^T += V^T . P^T -------------------------------------------------------------------------------------------
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq) o[nq][dt] = mfma16(vreg[dt], plow[nq], mfma16(vreg[dt], preg[nq], o[nq][dt]));
  };

  // One turn: fetch this step's values and (PIPE) the next step's keys, then compute the step on `cur`.
  auto turn = [&](int base, uintx4 (&cur)[2][KT], uintx4 (&next)[PIPE ? 2 : 1][PIPE ? KT : 1]) {
    const bool here = inside(base);
    if constexpr (!PIPE) {
      if (here) load_keys(base, cur, unchecked);
      else load_keys(base, cur, checked);
    }
    // memory first: this step's values (needed after the softmax) and the next step's keys (needed next turn)
    if (here) load_values(base, vreg, unchecked);
    else load_values(base, vreg, checked);
    if constexpr (PIPE) {
      if (base + 32 <= range_hi) {
        if (inside(base + 32)) load_keys(base + 32, next, unchecked);
        else load_keys(base + 32, next, checked);
      }
    }
    if constexpr (FRESH) {
      if (owns_new && base == (new_pos & ~31)) {  // the new key and value take the place of what the page holds
        const int at = new_pos - base;
#pragma unroll
        for (int j = 0; j < 2; ++j)
          if (key_in_step + j * 4 == at) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) cur[j][kt] = knew[kt];
          }
        if (g == (at >> 3)) {
          const int word = (at & 7) >> 1, shift = (at & 1) * 16;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int w = 0; w < 4; ++w)
              if (w == word) vreg[dt][w] = (vreg[dt][w] & ~(0xffffu << shift)) | (vnew[dt] << shift);
        }
      }
    }
    // every valid column sees the whole step: below the diagonal, inside window and segment
    const bool whole = here && base + 31 <= t.first_pos && (a.window == 0 || base >= last_pos - a.window + 1);
    if (whole) step(base, cur, unchecked);
    else step(base, cur, checked);
  };
  const int first_base = range_lo & ~31;
  if constexpr (PIPE) {
    if (first_base <= range_hi) {
      if (inside(first_base)) load_keys(first_base, kreg, unchecked);
      else load_keys(first_base, kreg, checked);
    }
    if constexpr (FRESH) encode_fresh();  // while the first keys are on their way
    for (int base = first_base; base <= range_hi; base += 64) {  // two turns: the key registers swap roles
      turn(base, kreg, knext);
      if (base + 32 > range_hi) break;
      turn(base + 32, knext, kreg);
    }
  } else {
    if constexpr (FRESH) encode_fresh();
    for (int base = first_base; base <= range_hi; base += 32) turn(base, kreg, knext);
  }

  // ---- results: lane holds, per column, dims dt * 16 + 4g .. + 3 ------------------------------------------------------
  const float nan = __uint_as_float(0x7fc00000u);
  poisoned = __any(poisoned);
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    l[nq] += __shfl_xor(l[nq], 16, 64);
    l[nq] += __shfl_xor(l[nq], 32, 64);
    if (SPLIT) {
      if (!col_valid[nq]) continue;  // (next column) the merge never reads columns that are no (token, head) pair
      const int c = nq * 16 + r16;
      float* dst = a.partial + (part * (16 * NQ) + c) * PSTRIDE;
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
        uintx2 packed;
        packed.x = bf16_pair(o[nq][dt][0] * inv, o[nq][dt][1] * inv);
        packed.y = bf16_pair(o[nq][dt][2] * inv, o[nq][dt][3] * inv);
        *reinterpret_cast<uintx2*>(a.out + col_at[nq] + dt * 16 + g * 4) = packed;
      }
    }
  }
  }  // pass
}

template <int NQ, bool SPLIT, bool PIPE, bool FRESH, bool ONCE>
__global__ __launch_bounds__(64, (SPLIT && NQ == 1 && D <= 128) ? 2 : 1) void attention_mfma_kernel(const Args a) {
  attention_mfma_body<NQ, SPLIT, PIPE, FRESH, ONCE>(
      a, Where{static_cast<int>(blockIdx.x), static_cast<int>(blockIdx.y), static_cast<int>(blockIdx.z),
               static_cast<int>(gridDim.x), static_cast<int>(gridDim.y), static_cast<int>(threadIdx.x)});
}

// ---- prompt portions: four waves share every key and value through LDS ------------------------------------------------
// A block of 4 waves works on 4 consecutive tiles of one request and one kv head (4 * 16 * NQ columns).  The keys and
// values of a step of 32 keys are fetched from the pages ONCE per block - every thread moves a few 16-byte pieces into
// LDS, double-buffered, one barrier per step - and each wave reads its MFMA A operands from there.  Against one wave
// per tile this takes three quarters of the traffic off the vector memory pipe and the address arithmetic off the
// waves.  With 16 columns per wave (NQ = 1) three blocks fit a compute unit; with 32 (NQ = 2) two, which do a step for
// twice the columns with the same loads, barriers and bookkeeping - the host takes them where they still fill the
// device.  In LDS a key row is stored at the MFMA row it feeds (tile j, row rho); a value row is one dim's 32 keys.
// Pages must hold at least 8 tokens (an aligned run of 8 keys of a value row is one 16-byte piece).
constexpr int kSharedWaves = 4;
// Rows in LDS, in bfloat16.  16 lanes read 16 bytes each from 16 consecutive rows; such a read runs at full rate when
// the rows are 2 (mod 4) pieces of 16 bytes apart (measured: 1.5 times slower with an odd number of pieces, worse
// with a multiple of 4), so rows are padded up to that: keys 2 * D bytes + 0 or 32, values 64 bytes + 32.
constexpr int KROW = D + ((D / 8) % 4 == 2 ? 0 : 16);
constexpr int VROW = 32 + 16;
constexpr float kLazy = 8.f;  // the exponentials' reference point trails the maximum by at most 2^kLazy

// SP: pages per step of 32 keys (4: pages of 8 tokens, 2: of 16, 1: of 32 or more) - with it the page arithmetic of a
// step is known when compiling.
template <int NQ, int SP>
__device__ __forceinline__ void attention_shared_body(const Args& a, const int block, const int thread) {
  const int page_shift = SP == 4 ? 3 : (SP == 2 ? 4 : a.page_shift);
  __shared__ __align__(16) bf16_t k_lds[2][32 * KROW];
  __shared__ __align__(16) bf16_t v_lds[2][D * VROW];
  __shared__ int bad_page;
  const int tid = thread, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Late tiles of a prompt see the most keys.  Blocks are ranked longest first, and the ranks are dealt out to the
  // compute units like cards in a snake: the first `units` blocks take the longest, the next `units` blocks the
  // following ranks in ascending order, so that the two blocks that share a unit add up to about the same work.
  const int heads = a.kv_heads * a.head_groups, round = 2 * a.units;
  const int turn = block / round, within = block % round;
  const int total = a.tiles * heads, in_round = min(round, total - turn * round);
  // a short last round has in_round < round blocks: its second part, if any, mirrors onto the ranks that exist
  const int rank = turn * round + (within < a.units ? within : in_round - 1 - (within - a.units));
  Tile t = find_tile(a, a.tiles - 1 - rank / heads, kSharedWaves * a.tokens_per_tile);
  if (!t.found) return;  // the same in every wave of the block
  t.request = __builtin_amdgcn_readfirstlane(t.request);  // the same in every lane: addresses built on it stay scalar
  t.first_row = __builtin_amdgcn_readfirstlane(t.first_row);
  t.tokens = __builtin_amdgcn_readfirstlane(t.tokens);
  t.first_pos = __builtin_amdgcn_readfirstlane(t.first_pos);
  const int kvh = (rank % heads) / a.head_groups, hg = (rank % heads) % a.head_groups;
  const uintx4 zero = uintx4{0u, 0u, 0u, 0u};
  const int page_mask = (1 << page_shift) - 1;
  if (tid == 0) bad_page = 0;

  // this wave's tile inside the block's, and this lane's columns
  const int wave_token0 = wave * a.tokens_per_tile;
  const bool wave_active = wave_token0 < t.tokens;
  const int wave_first_pos = t.first_pos + wave_token0;
  const int wave_last_pos = t.first_pos + min(t.tokens, wave_token0 + a.tokens_per_tile) - 1;
  bool col_valid[NQ];
  int col_pos[NQ], col_low[NQ];
  long col_at[NQ];
  uintx4 qreg[NQ][KT];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const int c = nq * 16 + r16;
    const int token = wave_token0 + c / a.heads_per_tile, head_in_group = hg * a.heads_per_tile + c % a.heads_per_tile;
    col_valid[nq] = token < t.tokens && c / a.heads_per_tile < a.tokens_per_tile && head_in_group < a.group;
    col_pos[nq] = t.first_pos + token;
    col_low[nq] = a.window > 0 ? max(0, col_pos[nq] - a.window + 1) : 0;
    col_at[nq] = (static_cast<long>(t.first_row + token) * a.q_heads + kvh * a.group + head_in_group) * D;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      const int dim = kt * 32 + g * 8;
      qreg[nq][kt] = (col_valid[nq] && dim < D) ? *reinterpret_cast<const uintx4*>(a.q + col_at[nq] + dim) : zero;
    }
  }
  // keys the block looks at
  const int last_pos = t.first_pos + t.tokens - 1;
  const int range_lo = a.window > 0 ? max(0, t.first_pos - a.window + 1) : 0;
  const int range_hi = last_pos;

  // The sum of a column's weights is accumulated by the matrix cores from the weights as they enter the weighted
  // sum: numerator and denominator carry the same rounding, and no lane has to add its keys up.
  const uintx4 ones = uintx4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  float m[NQ];
  floatx4 l[NQ], o[NQ][DT];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    m[nq] = col_valid[nq] ? -INFINITY : 1e30f;  // (a column that is no (token, head) pair: all its weights are 0)
    l[nq] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[nq][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- the block's loads: pieces of 16 bytes, piece p * 256 + tid ------------------------------------------------------
  const int* table = a.block_table + static_cast<long>(a.table_rows != nullptr ? a.table_rows[t.request] : t.request) * a.table_width;
  const char* k_bytes = reinterpret_cast<const char*>(a.k_pages);
  const char* v_bytes = reinterpret_cast<const char*>(a.v_pages);
  const uint32_t page_bytes = static_cast<uint32_t>(a.kv_heads) * D * 2u << page_shift;
  const uint32_t head_bytes = static_cast<uint32_t>(kvh) * D * 2u << page_shift;
  constexpr int kKeyPieces = 32 * (D / 8), kValuePieces = D * 4;
  constexpr int PK = (kKeyPieces + 255) / 256, PV = (kValuePieces + 255) / 256;
  const int run_shift = min(2, page_shift - 3);  // aligned runs of 8 keys of this step in one page row: 1, 2 or 4
  const std::true_type checked{};
  const std::false_type unchecked{};
  bool bad = false;
  // What a thread moves does not change from step to step: which key of the step and which 16 bytes of its row
  // (keys), which dim and which run of 8 keys (values), which of the step's pages that is, and where the piece goes
  // in LDS.  What changes - the step's 1, 2 or 4 page ids - is the same for every thread: it is read and checked with
  // scalar instructions, one step before the loads that need it are issued, so no load waits for the table entry
  // that addresses it and no lane spends arithmetic on it.
  constexpr int step_pages = SP, span = 32 / SP;  // (span: keys of a step in one page)
  int k_sel[PK], v_sel[PV];             // which of the step's pages holds the piece
  uint32_t k_from[PK], v_from[PV];      // byte offset inside the page, without what the step's first key adds
  uint32_t k_to[PK], v_to[PV];          // element offset in the LDS buffer
  bool k_mine[PK], v_mine[PV];
#pragma unroll
  for (int p = 0; p < PK; ++p) {
    const int c = p * 256 + tid, key = c / (D / 8);
    k_mine[p] = kKeyPieces % 256 == 0 || c < kKeyPieces;  // (known when compiling for the usual head sizes)
    k_sel[p] = step_pages == 1 ? 0 : key >> page_shift;
    k_from[p] = head_bytes + (c % (D / 8)) * 16u + static_cast<uint32_t>(key & page_mask) * (D * 2u);
    k_to[p] = (((key >> 2) & 1) * 16 + (key >> 3) * 4 + (key & 3)) * KROW + (c % (D / 8)) * 8;  // tile j, row rho
  }
#pragma unroll
  for (int p = 0; p < PV; ++p) {
    const int c = p * 256 + tid;
    const int run = (c / D) >> run_shift, within = c - ((run * D) << run_shift);
    const int dim = within >> run_shift, piece = (run << run_shift) + (within & ((1 << run_shift) - 1));
    v_mine[p] = kValuePieces % 256 == 0 || c < kValuePieces;
    v_sel[p] = step_pages == 1 ? 0 : (piece * 8) >> page_shift;
    v_from[p] = head_bytes + (static_cast<uint32_t>(dim) << (page_shift + 1)) + static_cast<uint32_t>((piece * 8) & page_mask) * 2u;
    v_to[p] = dim * VROW + piece * 8;
  }
  // With the usual sizes (a head of 128 and pages of 16 or more, say) all pieces that the wave moves in one turn p
  // come from the same page of the step.  Then the page's address stays in scalar registers and a load takes the
  // thread's constant 32-bit offset beside it: no address arithmetic per lane and step.
  int k_page[PK], v_page[PV];
  bool same_page = true;
#pragma unroll
  for (int p = 0; p < PK; ++p) {
    k_page[p] = __builtin_amdgcn_readfirstlane(k_sel[p]);
    same_page = same_page && (k_sel[p] == k_page[p] || !k_mine[p]);
  }
#pragma unroll
  for (int p = 0; p < PV; ++p) {
    v_page[p] = __builtin_amdgcn_readfirstlane(v_sel[p]);
    same_page = same_page && (v_sel[p] == v_page[p] || !v_mine[p]);
  }
  same_page = __all(same_page);
  // key of a piece relative to the step's first: only steps at the edge of the range ask, so it is not kept
  auto k_key = [&](int p) { return (p * 256 + tid) / (D / 8); };
  auto v_key = [&](int p) {
    const int c = p * 256 + tid, run = (c / D) >> run_shift, within = c - ((run * D) << run_shift);
    return ((run << run_shift) + (within & ((1 << run_shift) - 1))) * 8;
  };
  // The page ids of the step at `base`.  CHECK: the step may reach outside [range_lo, range_hi]; pages wholly
  // outside are not looked up (their entries may lie beyond the table).
  auto page_wanted = [&](int base, int i) {
    const int first = base + (i << page_shift);
    return first <= range_hi && first + span - 1 >= range_lo;
  };
  auto lookup = [&](int base, int (&pages)[4], auto check) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pages[i] = 0;
      if (i < step_pages && (!decltype(check)::value || page_wanted(base, i))) pages[i] = table[(base >> page_shift) + i];
    }
  };
  auto fetch = [&](int base, const int (&pages)[4], uintx4 (&kst)[PK], uintx4 (&vst)[PV], auto check) {
    size_t at[4];  // byte offset of each of the step's pages
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int page = pages[i];
      if (i < step_pages && (!decltype(check)::value || page_wanted(base, i)) && (page < 0 || page >= a.num_pages)) {
        bad = true;
        page = 0;
      }
      at[i] = static_cast<size_t>(page) * page_bytes;
    }
    auto of = [&](int sel) { return sel == 0 ? at[0] : (sel == 1 ? at[1] : (sel == 2 ? at[2] : at[3])); };
    const uint32_t in_page = static_cast<uint32_t>(base & page_mask);  // pages of more than 32 tokens: where the step begins
#pragma unroll
    for (int p = 0; p < PK; ++p) {
      bool wanted = k_mine[p];
      if (decltype(check)::value) {
        const int key = base + k_key(p);
        wanted = wanted && key >= range_lo && key <= range_hi;
      }
      kst[p] = zero;
      if (wanted) {
        if (same_page) kst[p] = *reinterpret_cast<const uintx4*>(k_bytes + of(k_page[p]) + in_page * (D * 2u) + k_from[p]);
        else kst[p] = *reinterpret_cast<const uintx4*>(k_bytes + of(k_sel[p]) + in_page * (D * 2u) + k_from[p]);
      }
    }
#pragma unroll
    for (int p = 0; p < PV; ++p) {
      int live = 8;
      bool wanted = v_mine[p];
      if (decltype(check)::value) {
        const int key = base + v_key(p);
        live = min(8, range_hi - key + 1);
        wanted = wanted && live > 0 && key + 7 >= range_lo;
      }
      uintx4 v = zero;
      if (wanted) {
        if (same_page) v = *reinterpret_cast<const uintx4*>(v_bytes + of(v_page[p]) + in_page * 2u + v_from[p]);
        else v = *reinterpret_cast<const uintx4*>(v_bytes + of(v_sel[p]) + in_page * 2u + v_from[p]);
        if (decltype(check)::value && live < 8) {  // slots beyond the last key were never written: anything, NaN included
          uint32_t keep[4];
#pragma unroll
          for (int w = 0; w < 4; ++w) keep[w] = live >= 2 * w + 2 ? 0xffffffffu : (live == 2 * w + 1 ? 0x0000ffffu : 0u);
          v = uintx4{v.x & keep[0], v.y & keep[1], v.z & keep[2], v.w & keep[3]};
        }
      }
      vst[p] = v;
    }
  };
  // The same for a step that lies inside the range as a whole, when every turn's pieces come from one page: the
  // page's address is scalar, a load adds the thread's constant offset, and nothing is tested per piece.
  auto fetch_inside = [&](int base, const int (&pages)[4], uintx4 (&kst)[PK], uintx4 (&vst)[PV]) {
    size_t at[SP];
#pragma unroll
    for (int i = 0; i < SP; ++i) {
      int page = pages[i];
      if (static_cast<uint32_t>(page) >= static_cast<uint32_t>(a.num_pages)) {
        bad = true;
        page = 0;
      }
      at[i] = static_cast<size_t>(page) * page_bytes;
    }
    auto of = [&](int sel) {
      if constexpr (SP == 1) return at[0];
      else if constexpr (SP == 2) return sel == 0 ? at[0] : at[1];
      else return sel == 0 ? at[0] : (sel == 1 ? at[1] : (sel == 2 ? at[2] : at[3]));
    };
    const uint32_t in_page = SP == 1 ? static_cast<uint32_t>(base & page_mask) : 0u;
#pragma unroll
    for (int p = 0; p < PK; ++p) {
      kst[p] = zero;
      if (k_mine[p]) kst[p] = *reinterpret_cast<const uintx4*>(k_bytes + of(k_page[p]) + in_page * (D * 2u) + k_from[p]);
    }
#pragma unroll
    for (int p = 0; p < PV; ++p) {
      vst[p] = zero;
      if (v_mine[p]) vst[p] = *reinterpret_cast<const uintx4*>(v_bytes + of(v_page[p]) + in_page * 2u + v_from[p]);
    }
  };
  auto stash = [&](int buffer, const uintx4 (&kst)[PK], const uintx4 (&vst)[PV]) {
#pragma unroll
    for (int p = 0; p < PK; ++p)
      if (k_mine[p]) *reinterpret_cast<uintx4*>(&k_lds[buffer][k_to[p]]) = kst[p];
#pragma unroll
    for (int p = 0; p < PV; ++p)
      if (v_mine[p]) *reinterpret_cast<uintx4*>(&v_lds[buffer][v_to[p]]) = vst[p];
  };

  // ---- the parts of a step of 32 keys -----------------------------------------------------------------------------------
  // scores: S^T = K . Q^T from the keys in LDS
  auto scores = [&](int buffer, floatx4 (&s)[NQ][2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq) s[nq][j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const bool inside = (D % 32 == 0) || kt * 32 + g * 8 < D;
        const uintx4 keys = inside ? *reinterpret_cast<const uintx4*>(&k_lds[buffer][(j * 16 + r16) * KROW + kt * 32 + g * 8])
                                   : zero;
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq) s[nq][j] = mfma16(keys, qreg[nq][kt], s[nq][j]);
      }
    }
  };
  // keys that a column does not see count as -inf
  auto hide = [&](int base, floatx4 (&s)[NQ][2]) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = base + g * 8 + j * 4 + i;
          const bool seen = col_valid[nq] && key <= col_pos[nq] && key >= col_low[nq];
          if (!seen) s[nq][j][i] = -INFINITY;
        }
  };
  // The reference point of the exponentials follows the maximum lazily: it moves only when the maximum has grown by
  // more than 2^kLazy, so weights stay below 2^kLazy (harmless in float32 sums, and bfloat16 keeps its relative
  // precision) and the accumulators are rescaled a few times per row instead of at every step.  Returns whether
  // some column's reference moved; `correction` is what its accumulators are to be multiplied by then.
  auto follow = [&](const floatx4 (&s)[NQ][2], float (&correction)[NQ]) {
    bool rescale = false;
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      float top = fmaxf(fmaxf(fmaxf(s[nq][0][0], s[nq][0][1]), fmaxf(s[nq][0][2], s[nq][0][3])),
                        fmaxf(fmaxf(s[nq][1][0], s[nq][1][1]), fmaxf(s[nq][1][2], s[nq][1][3])));
      top = max_over_groups(top);
      const float scaled = top * a.scale_log2;                 // the scale is positive: max commutes with it
      const bool moved = scaled > m[nq] + kLazy;               // also the first keys seen: m is -inf
      const float m_new = moved ? scaled : m[nq];
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;   // nothing seen yet: every weight is 0, no NaN
      correction[nq] = moved ? __builtin_amdgcn_exp2f(m[nq] - m_safe) : 1.f;
      rescale = rescale || moved;
      m[nq] = m_new;
    }
    return __any(rescale);
  };
  auto rescale = [&](const float (&correction)[NQ]) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      l[nq] *= correction[nq];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[nq][dt] *= correction[nq];
    }
  };
  // Exponents of the weights, base 2, relative to the reference point.
  auto exponents = [&](const floatx4 (&s)[NQ][2], float (&t)[NQ][8]) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      const float m_safe = m[nq] == -INFINITY ? 0.f : m[nq];   // nothing seen yet: every weight is 0, no NaN
#pragma unroll
      for (int e = 0; e < 8; ++e) t[nq][e] = fmaf(s[nq][e >> 2][e & 3], a.scale_log2, -m_safe);
    }
  };
  // A weight enters the second product as two bfloat16 numbers (p = high + low, 16 bits of mantissa together), so
  // that the weighted sum does not carry the 2^-9 relative error of a single bfloat16.
  auto weights = [&](const float (&t)[NQ][8], uintx4 (&preg)[NQ], uintx4 (&plow)[NQ]) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      uint32_t high[4], low[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const floatx2 p = {__builtin_amdgcn_exp2f(t[nq][2 * e]), __builtin_amdgcn_exp2f(t[nq][2 * e + 1])};
        high[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2));
        const floatx2 rest = {p[0] - __uint_as_float(high[e] << 16), p[1] - __uint_as_float(high[e] & 0xffff0000u)};
        low[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2));
      }
      preg[nq] = uintx4{high[0], high[1], high[2], high[3]};
      plow[nq] = uintx4{low[0], low[1], low[2], low[3]};
    }
  };
  // O^T += V^T . P^T, and the weights' sums from the same two-part weights: a row of ones beside the value rows
  auto accumulate = [&](int buffer, const uintx4 (&preg)[NQ], const uintx4 (&plow)[NQ]) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) l[nq] = mfma16(ones, plow[nq], mfma16(ones, preg[nq], l[nq]));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const uintx4 values = *reinterpret_cast<const uintx4*>(&v_lds[buffer][(dt * 16 + r16) * VROW + g * 8]);
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq) o[nq][dt] = mfma16(values, plow[nq], mfma16(values, preg[nq], o[nq][dt]));
    }
  };
  // One step.  MASK: some column does not see the whole step.
  // Without a mask the maximum is not looked for at all as long as no exponent of the wave exceeds kLazy: then no
  // reference point would move, and the exponents are the ones the weights need.  (A column that has seen nothing
  // yet has the reference -inf and asks for the search; columns that are no (token, head) pair start with a huge
  // reference and never ask.)
  auto step = [&](int base, int buffer, auto mask) {
    floatx4 s[NQ][2];
    float t[NQ][8], correction[NQ];
    uintx4 preg[NQ], plow[NQ];
    scores(buffer, s);
    if (decltype(mask)::value) {
      hide(base, s);
      if (follow(s, correction)) rescale(correction);
      exponents(s, t);
    } else {
      exponents(s, t);
      bool search = false;
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq) {
        const float top = fmaxf(fmaxf(fmaxf(t[nq][0], t[nq][1]), fmaxf(t[nq][2], t[nq][3])),
                                fmaxf(fmaxf(t[nq][4], t[nq][5]), fmaxf(t[nq][6], t[nq][7])));
        search = search || top > kLazy || m[nq] == -INFINITY;
      }
      if (__any(search)) {
        if (follow(s, correction)) rescale(correction);
        exponents(s, t);
      }
    }
    weights(t, preg, plow);
    accumulate(buffer, preg, plow);
  };

  uintx4 kst[PK], vst[PV];
  int pages[4];
  const int first_base = range_lo & ~31;
  auto inside = [&](int base) { return base >= range_lo && base + 31 <= range_hi; };
  auto lookup_step = [&](int base) {
    if (inside(base)) lookup(base, pages, unchecked);
    else lookup(base, pages, checked);
  };
  auto fetch_step = [&](int base) {
    if (inside(base)) fetch(base, pages, kst, vst, unchecked);
    else fetch(base, pages, kst, vst, checked);
  };
  lookup_step(first_base);
  fetch_step(first_base);
  if (first_base + 32 <= range_hi) lookup_step(first_base + 32);
  stash(0, kst, vst);
  __syncthreads();
  // Steps before `calm_to` (and from `calm_from` on, with a window) are calm: the step, the next one that is
  // fetched meanwhile and the one after it whose pages are looked up all lie inside the range, and every wave sees
  // all 32 keys - nothing is tested in them.
  const int calm_from = a.window > 0 ? (max(range_lo, last_pos - a.window + 1) + 31) & ~31 : first_base;
  // base < calm_to: base + 95 <= range_hi, and base + 31 <= the block's first position
  const int calm_to = same_page ? min(range_hi - 94, t.first_pos - 30) : first_base;
  // Three loops, one after the other, instead of one with a test per step: steps before the calm ones (a window's
  // first steps), the calm ones, and those after.  In a loop of its own the calm step's sums stay in their registers
  // from step to step (in a loop shared with the other kinds of step the compiler copied all of them at every turn);
  // a wave without tokens runs the same loops without the arithmetic.
  int buffer = 0, base = first_base;
  auto ordinary_step = [&](int base, int buffer) {
    const bool more = base + 32 <= range_hi;
    if (more) fetch_step(base + 32);
    if (base + 64 <= range_hi) lookup_step(base + 64);
    // the wave's tokens see some key of this step
    if (wave_active && base <= wave_last_pos && (a.window == 0 || base + 31 >= wave_first_pos - a.window + 1)) {
      const bool whole = base >= range_lo && base + 31 <= wave_first_pos &&
                         (a.window == 0 || base >= wave_last_pos - a.window + 1);
      if (whole) step(base, buffer, unchecked);
      else step(base, buffer, checked);
    }
    if (more) stash(buffer ^ 1, kst, vst);
    __syncthreads();
  };
  for (; base <= range_hi && base < calm_from; base += 32, buffer ^= 1) ordinary_step(base, buffer);
  if (wave_active) {
    for (; base < calm_to; base += 32, buffer ^= 1) {
      fetch_inside(base + 32, pages, kst, vst);
      lookup(base + 64, pages, unchecked);
      step(base, buffer, unchecked);
      stash(buffer ^ 1, kst, vst);
      __syncthreads();
    }
  } else {
    for (; base < calm_to; base += 32, buffer ^= 1) {
      fetch_inside(base + 32, pages, kst, vst);
      lookup(base + 64, pages, unchecked);
      stash(buffer ^ 1, kst, vst);
      __syncthreads();
    }
  }
  for (; base <= range_hi; base += 32, buffer ^= 1) ordinary_step(base, buffer);
  if (bad) bad_page = 1;
  __syncthreads();
  const bool poisoned = bad_page != 0;
  const float nan = __uint_as_float(0x7fc00000u);
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    if (!col_valid[nq]) continue;
    const float inv = poisoned ? nan : 1.f / l[nq][0];  // every row of the ones tile holds the column's sum
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uintx2 packed;
      packed.x = bits_by_integer_rounding(o[nq][dt][0] * inv) | (bits_by_integer_rounding(o[nq][dt][1] * inv) << 16);
      packed.y = bits_by_integer_rounding(o[nq][dt][2] * inv) | (bits_by_integer_rounding(o[nq][dt][3] * inv) << 16);
      *reinterpret_cast<uintx2*>(a.out + col_at[nq] + dt * 16 + g * 4) = packed;
    }
  }
}

template <int NQ, int SP>
__global__ __launch_bounds__(64 * kSharedWaves, D <= 128 ? (NQ == 1 ? 3 : 2) : 1) void attention_shared_kernel(const Args a) {
  attention_shared_body<NQ, SP>(a, static_cast<int>(blockIdx.x), static_cast<int>(threadIdx.x));
}

// ---- single tokens and short prompt portions in one launch ---------------------------------------------------------------
// A step that decodes some requests and feeds a short portion of another's prompt has two attention launches that do
// not depend on each other and do not fill the device: the single tokens' keys stream from memory, the portion's few
// blocks wait for one load after the other.  One after the other they take the sum of their times; on two streams
// they run beside each other, and the two waits between the streams cost most of what that saves.  Here they are one
// grid: the first `portion_blocks` blocks are the portion's (they walk the longest, so they start first), every block
// after them is four independent waves of the single tokens' kernel, wave w of block b standing where block
// 4 b + w of that kernel's own grid (kv heads x items of the plan) would.  The text of either kernel is the same as in
// its own launch, so the bits are.  Registers are the larger of the two (two waves a SIMD, which the single tokens'
// kernel has anyway); every block holds the portion kernel's LDS.
template <bool ONCE, int SP>
__global__ __launch_bounds__(64 * kSharedWaves, 2) void attention_pair_kernel(const Args single, const Args portion,
                                                                              const int portion_blocks) {
  if constexpr (D % 64 == 0) {
    if (static_cast<int>(blockIdx.x) < portion_blocks) {
      attention_shared_body<1, SP>(portion, static_cast<int>(blockIdx.x), static_cast<int>(threadIdx.x));
    } else {
      const int gx = single.kv_heads * single.head_groups, gy = single.items_grid;
      const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
      const int unit = (static_cast<int>(blockIdx.x) - portion_blocks) * kSharedWaves + wave;
      if (unit >= gx * gy) return;
      attention_mfma_body<1, true, true, true, ONCE>(single, Where{unit % gx, unit / gx, 0, gx, gy, static_cast<int>(threadIdx.x) & 63});
    }
  }
}

// Merge of the segments' partial results: out = sum_z 2^(m_z - M) O_z / sum_z 2^(m_z - M) l_z, M = max_z m_z
// (csrc/paged_decode.cu:528-544 of the reference has the same rule in base e).  One block of kMergeWaves waves per
// (tile, head group, column); a lane owns dims lane, lane + 64, ...; wave w sums the segments w, w + kMergeWaves, ...
// in ascending order, and the waves' sums are added in the order of the waves: the order of the whole sum is fixed.
constexpr int kMergeWaves = 4;

template <int NQ>
__global__ __launch_bounds__(64 * kMergeWaves) void attention_merge_kernel(const Args a) {
  constexpr int PER = (D + 63) / 64;
  __shared__ float sums[kMergeWaves][PER * 64 + 1];  // per wave: the weighted sum per dim, then the denominator
  Tile t{};
  if (a.plan != nullptr) {   // single tokens cut by a plan: block x is request seq_first + x, one row each
    t.found = true;
    t.tokens = 1;
    t.first_row = a.q_start[a.seq_first] + static_cast<int>(blockIdx.x);
  } else {
    t = find_tile(a, blockIdx.x, a.tokens_per_tile);
    if (!t.found) return;
  }
  const int kvh = blockIdx.y / a.head_groups, hg = blockIdx.y % a.head_groups;
  const int c = blockIdx.z, lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int token = c / a.heads_per_tile, head_in_group = hg * a.heads_per_tile + c % a.heads_per_tile;
  if (token >= t.tokens || head_in_group >= a.group) return;
  // the request's partial results: `splits` tiles, `split_stride` floats apart
  const float* src = a.partial + (((static_cast<long>(blockIdx.x) * gridDim.y + blockIdx.y) * a.num_splits) * (16 * NQ) + c) * PSTRIDE;
  long split_stride = static_cast<long>(16 * NQ) * PSTRIDE;
  int splits = a.num_splits;
  if (a.plan != nullptr) {  // the plan's items of request blockIdx.x follow each other
    splits = a.plan[5 + 2 * blockIdx.x];
    src = a.partial + ((static_cast<long>(a.plan[4 + 2 * blockIdx.x]) * gridDim.y + blockIdx.y) * (16 * NQ) + c) * PSTRIDE;
    split_stride *= gridDim.y;
  }
  // this wave's segments: z = wave + kMergeWaves * i.  Eight segments' loads go out together; the first eight are
  // asked for before the maxima - they do not depend on them, and the kernel is a chain of trips to memory.
  const int mine = (splits - wave + kMergeWaves - 1) / kMergeWaves;
  auto fetch8 = [&](int i0, int ii0, int count, float (&v)[8][PER]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float* p = src + (wave + static_cast<long>(kMergeWaves) * (i0 + min(ii0 + j, count - 1))) * split_stride;
#pragma unroll
      for (int e = 0; e < PER; ++e) v[j][e] = lane + e * 64 < D ? p[lane + e * 64] : 0.f;
    }
  };
  float ahead[8][PER] = {};
  if (mine > 0) fetch8(0, 0, min(64, mine), ahead);
  // every wave finds the maximum over all segments (a lane per segment).  A segment's maximum and sum are asked for
  // together and whatever the lane (a lane beyond the last segment reads the last one's): the first 64 segments'
  // are handed to the lanes that weigh them by a shuffle instead of a second trip to memory.
  float top = -INFINITY, first_m = -INFINITY, first_l = 0.f;
  bool poisoned = false;
  for (int z0 = 0; z0 < splits; z0 += 64) {
    const int z = z0 + lane;
    const long at = static_cast<long>(max(0, min(z, splits - 1))) * split_stride;
    float mz = src[at + D];
    const float lz = src[at + D + 1];
    if (z >= splits) mz = -INFINITY;
    if (z0 == 0) first_m = mz, first_l = lz;
    poisoned = poisoned || mz != mz;
    top = fmaxf(top, mz);
  }
  top = wave_max(top);
  poisoned = __any(poisoned);
  float denom = 0.f, acc[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) acc[i] = 0.f;
  for (int i0 = 0; i0 < mine; i0 += 64) {
    const int i = i0 + lane;
    float w = 0.f;
    const long z = wave + static_cast<long>(kMergeWaves) * i;
    float mz = __shfl(first_m, static_cast<int>(z & 63), 64), lz = __shfl(first_l, static_cast<int>(z & 63), 64);
    if (i < mine && z >= 64) {
      mz = src[z * split_stride + D];
      lz = src[z * split_stride + D + 1];
    }
    if (i < mine) {
      w = (mz == -INFINITY || mz != mz) ? 0.f : __builtin_amdgcn_exp2f(mz - top);
      denom += w * lz;
    }
    const int count = min(64, mine - i0);
    for (int ii0 = 0; ii0 < count; ii0 += 8) {  // ascending segments
      float v[8][PER];
      if (i0 == 0 && ii0 == 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int e = 0; e < PER; ++e) v[j][e] = ahead[j][e];
      } else {
        fetch8(i0, ii0, count, v);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float wz = ii0 + j < count ? __shfl(w, ii0 + j, 64) : 0.f;
#pragma unroll
        for (int e = 0; e < PER; ++e) acc[e] = fmaf(wz, v[j][e], acc[e]);
      }
    }
  }
  denom = wave_sum(denom);
#pragma unroll
  for (int e = 0; e < PER; ++e) sums[wave][e * 64 + lane] = acc[e];
  if (lane == 0) sums[wave][PER * 64] = denom;
  __syncthreads();
  if (wave != 0) return;
  float total = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) acc[e] = 0.f;
  for (int w = 0; w < kMergeWaves; ++w) {
    total += sums[w][PER * 64];
#pragma unroll
    for (int e = 0; e < PER; ++e) acc[e] += sums[w][e * 64 + lane];
  }
  bf16_t* dst = a.out + (static_cast<long>(t.first_row + token) * a.q_heads + kvh * a.group + head_in_group) * D;
  const float inv = poisoned ? __uint_as_float(0x7fc00000u) : 1.f / total;
#pragma unroll
  for (int e = 0; e < PER; ++e)
    if (lane + e * 64 < D) dst[lane + e * 64] = from_float<bf16_t>(acc[e] * inv);
}

template <int NQ>
int launch(const Args& a, int tiles, bool shared, hipStream_t stream) {
  dim3 grid(tiles, a.kv_heads * a.head_groups, a.num_splits);
  if (shared) {
    const dim3 blocks(tiles * a.kv_heads * a.head_groups);
    if (a.page_shift >= 5) attention_shared_kernel<NQ, 1><<<blocks, 64 * kSharedWaves, 0, stream>>>(a);
    else if (a.page_shift == 4) attention_shared_kernel<NQ, 2><<<blocks, 64 * kSharedWaves, 0, stream>>>(a);
    else if (a.page_shift == 3) attention_shared_kernel<NQ, 4><<<blocks, 64 * kSharedWaves, 0, stream>>>(a);
    else return -2;
    return AKV_LAUNCH_STATUS();
  }
  const bool items = a.plan != nullptr;  // single tokens whose keys were cut on the device: always with the merge
  if (items) grid = dim3(a.kv_heads * a.head_groups, a.items_grid, 1);
  const int columns = a.heads_per_tile * (a.single_tokens ? 1 : a.tokens_per_tile);   // that can be a (token, head) pair
  const dim3 merge_grid(items ? a.seq_count : tiles, a.kv_heads * a.head_groups, columns);
  auto merge = [&]() { attention_merge_kernel<NQ><<<merge_grid, 64 * kMergeWaves, 0, stream>>>(a); };
  if (a.num_splits == 1 && a.qkv == nullptr && !items) grid.x = (tiles + 1) / 2;  // a block takes a late tile and an early one
  // single tokens cut into segments: a key is read by one block per group of query heads - by one block where the
  // heads of a kv head fit one tile
  const bool once = a.single_tokens && a.head_groups == 1;
  if (a.qkv != nullptr) {
    if constexpr (NQ == 1 && D % 64 == 0) {
      if (!a.single_tokens) return -2;
      if (items || a.num_splits > 1) {
        if (once) attention_mfma_kernel<NQ, true, true, true, true><<<grid, 64, 0, stream>>>(a);
        else attention_mfma_kernel<NQ, true, true, true, false><<<grid, 64, 0, stream>>>(a);
        merge();
      } else {
        attention_mfma_kernel<NQ, false, true, true, false><<<grid, 64, 0, stream>>>(a);
      }
      return AKV_LAUNCH_STATUS();
    } else {
      return -2;
    }
  }
  if (items || a.num_splits > 1) {
    if (once) attention_mfma_kernel<NQ, true, true, false, true><<<grid, 64, 0, stream>>>(a);
    else attention_mfma_kernel<NQ, true, true, false, false><<<grid, 64, 0, stream>>>(a);
    merge();
  } else {
    attention_mfma_kernel<NQ, false, true, false, false><<<grid, 64, 0, stream>>>(a);
  }
  return AKV_LAUNCH_STATUS();
}

// The pair launch (see attention_pair_kernel), then the single tokens' merge.
int launch_pair(const Args& single, const Args& portion, int portion_tiles, hipStream_t stream) {
  if constexpr (D % 64 == 0) {
    const long portion_blocks = static_cast<long>(portion_tiles) * portion.kv_heads * portion.head_groups;
    const long units = static_cast<long>(single.kv_heads) * single.head_groups * single.items_grid;
    const long blocks = portion_blocks + (units + kSharedWaves - 1) / kSharedWaves;
    if (blocks > 0x7fffffffL) return -2;
    const bool once = single.head_groups == 1;
    const dim3 grid(static_cast<unsigned>(blocks));
    const int first = static_cast<int>(portion_blocks);
#define AKV_PAIR(SP_) \
    do { \
      if (once) attention_pair_kernel<true, SP_><<<grid, 64 * kSharedWaves, 0, stream>>>(single, portion, first); \
      else attention_pair_kernel<false, SP_><<<grid, 64 * kSharedWaves, 0, stream>>>(single, portion, first); \
    } while (0)
    if (portion.page_shift >= 5) AKV_PAIR(1);
    else if (portion.page_shift == 4) AKV_PAIR(2);
    else if (portion.page_shift == 3) AKV_PAIR(4);
    else return -2;
#undef AKV_PAIR
    const dim3 merge_grid(single.seq_count, single.kv_heads * single.head_groups, single.heads_per_tile);
    attention_merge_kernel<1><<<merge_grid, 64 * kMergeWaves, 0, stream>>>(single);
    return AKV_LAUNCH_STATUS();
  } else {
    return -2;
  }
}

// What every launch of a step shares, checked and put into `a`; 0 or an error code.
int common_args(Args& a, const void* q, const void* k_pages, const void* v_pages, void* out, const int* q_start,
                const int* seq_lens, const int* block_table, const int* table_rows, int table_width, int q_heads,
                int kv_heads, int page_size, long num_pages, float scale, int window) {
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  if (page_size < 4 || (1 << page_shift) != page_size || kv_heads <= 0 || q_heads % kv_heads != 0) return -2;
  a.q = static_cast<const bf16_t*>(q);
  a.k_pages = static_cast<const bf16_t*>(k_pages);
  a.v_pages = static_cast<const bf16_t*>(v_pages);
  a.out = static_cast<bf16_t*>(out);
  a.q_start = q_start;
  a.seq_lens = seq_lens;
  a.block_table = block_table;
  a.table_rows = table_rows;
  a.table_width = table_width;
  a.q_heads = q_heads;
  a.kv_heads = kv_heads;
  a.group = q_heads / kv_heads;
  a.page_shift = page_shift;
  a.num_pages = num_pages;
  a.scale_log2 = scale * kLog2e;
  a.window = window;
  a.units = 1;
  return 0;
}

// The compute units of the current device (asked once per device); 0 on an error.
int units_of_device() {
  static int units_of[64] = {0};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
  if (units_of[device] == 0) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0) return 0;
    units_of[device] = count;
  }
  return units_of[device];
}

}  // namespace

#define AKV_CONCAT2(a, b) a##b
#define AKV_CONCAT(a, b) AKV_CONCAT2(a, b)

// Attention of requests seq_first .. seq_first + seq_count - 1 of the step.  `nq` (1 or 2) sets the tile to
// 16 * nq query columns; `tiles` is the number of tiles over those requests (sum of ceil(tokens / tokens_per_tile));
// with num_splits > 1 `partial` must hold tiles * kv_heads * head_groups * num_splits * 16 * nq * (D + 4) floats.
// page_size must be a power of two, at least 4.  `single_tokens` says that every request brings exactly one token.
// `table_rows` (may be null): request r's pages are row table_rows[r] of `block_table` instead of row r - the table
// then is the engine's persistent one, a row per request slot.
// `shared`: blocks of four waves that share keys and values through LDS; `tiles` then counts tiles of
// 4 * tokens_per_tile tokens, num_splits must be 1 and pages hold at least 8 tokens.
// `plan` (not null: single tokens, at most 64 requests): seg_keys and num_splits are not used; the requests' keys were
// cut into items by akv_decode_plan with the same seq_first, seq_count and window; `items_grid` is the bound given
// there, and `partial` must hold items_grid * kv_heads * head_groups * 16 * nq * (D + 4) floats.
// `qkv` (not null: single tokens, nq 1, head sizes that are multiples of 64): the tokens' stacked raw projections
// [tokens, (q_heads + 2 * kv_heads) * D]; `q` is not read, the kernel norms (q_weight, k_weight, eps; both weights
// null: no norm) and rotates (rope_table [table_positions, D / 2, 2], null: no rotation) queries and the new keys
// itself and writes the new keys and values to the tokens' slots, which the block tables must already name.
extern "C" int AKV_CONCAT(akv_attention_mfma_d, AKV_HEAD_DIM)(
    const void* q, const void* k_pages, const void* v_pages, void* out, float* partial, const int* q_start,
    const int* seq_lens, const int* block_table, const int* table_rows, int table_width, int seq_first, int seq_count,
    int tiles, int nq,
    int q_heads, int kv_heads, int heads_per_tile, int head_groups, int tokens_per_tile, int page_size, long num_pages,
    float scale, int window, int seg_keys, int num_splits, int single_tokens, int shared, const void* qkv,
    const float* q_weight, const float* k_weight, float eps, const float* rope_table, int table_positions,
    const int* plan, int items_grid, hipStream_t stream) {
  if (tiles <= 0 || seq_count <= 0) return 0;
  if (heads_per_tile * tokens_per_tile > 16 * nq || kv_heads * head_groups > 65535 || num_splits > 65535 ||
      num_splits < 1 || (single_tokens && tiles != seq_count) || (shared && (page_size < 8 || num_splits != 1)) ||
      (qkv != nullptr && (shared || !single_tokens || nq != 1 || D % 64 != 0 || (q_weight == nullptr) != (k_weight == nullptr))) ||
      (plan != nullptr && (shared || !single_tokens || seq_count > 64 || items_grid < 1 || items_grid > 65535)))
    return -2;
  Args a;
  const int status = common_args(a, q, k_pages, v_pages, out, q_start, seq_lens, block_table, table_rows, table_width,
                                 q_heads, kv_heads, page_size, num_pages, scale, window);
  if (status != 0) return status;
  a.partial = partial;
  a.seq_first = seq_first;
  a.seq_count = seq_count;
  a.tiles = tiles;
  a.heads_per_tile = heads_per_tile;
  a.head_groups = head_groups;
  a.tokens_per_tile = tokens_per_tile;
  a.single_tokens = single_tokens;
  a.seg_keys = seg_keys;
  a.num_splits = num_splits;
  a.plan = plan;
  a.items_grid = items_grid;
  a.qkv = static_cast<const bf16_t*>(qkv);
  a.q_weight = q_weight;
  a.k_weight = k_weight;
  a.rope_table = rope_table;
  a.table_positions = table_positions;
  a.eps = eps;
  if (shared) {
    a.units = units_of_device();
    if (a.units == 0) return -3;
    if (static_cast<long>(tiles) * kv_heads * head_groups > 0x7fffffffL) return -2;
  }
  switch (nq) {
    case 1: return launch<1>(a, tiles, shared != 0, stream);
    case 2: return launch<2>(a, tiles, shared != 0, stream);
    default: return -2;
  }
}

// Single tokens and prompt portions of one step in ONE launch (see attention_pair_kernel), then the single tokens'
// merge.  The single tokens are requests single_first .. + single_count - 1 (at most 64), with their raw projections
// `qkv` and a plan of their keys as for the launch above with `qkv` and `plan` (so head sizes are multiples of 64);
// the portions are requests portion_first .. + portion_count - 1 in blocks of four tiles of 16 columns that share keys
// and values (`shared`, nq = 1; pages of 8 tokens and more), `portion_tiles` such blocks of tokens.  What the two
// write and read is as in their own launches.
extern "C" int AKV_CONCAT(akv_attention_pair_d, AKV_HEAD_DIM)(
    const void* q, const void* k_pages, const void* v_pages, void* out, const int* q_start, const int* seq_lens,
    const int* block_table, const int* table_rows, int table_width, int q_heads, int kv_heads, int page_size,
    long num_pages, float scale, int window,
    int single_first, int single_count, int single_heads_per_tile, int single_head_groups, float* partial,
    const int* plan, int items_grid, const void* qkv, const float* q_weight, const float* k_weight, float eps,
    const float* rope_table, int table_positions,
    int portion_first, int portion_count, int portion_tiles, int portion_heads_per_tile, int portion_head_groups,
    int portion_tokens_per_tile, hipStream_t stream) {
  if (single_count <= 0 || portion_count <= 0 || portion_tiles <= 0) return -2;
  if (D % 64 != 0 || page_size < 8 || single_count > 64 || plan == nullptr || qkv == nullptr || partial == nullptr ||
      items_grid < 1 || items_grid > 65535 || (q_weight == nullptr) != (k_weight == nullptr) ||
      single_heads_per_tile > 16 || portion_heads_per_tile * portion_tokens_per_tile > 16 ||
      kv_heads * single_head_groups > 65535)
    return -2;
  Args single, portion;
  int status = common_args(single, q, k_pages, v_pages, out, q_start, seq_lens, block_table, table_rows, table_width,
                           q_heads, kv_heads, page_size, num_pages, scale, window);
  if (status != 0) return status;
  portion = single;
  single.partial = partial;
  single.seq_first = single_first;
  single.seq_count = single_count;
  single.tiles = single_count;
  single.heads_per_tile = single_heads_per_tile;
  single.head_groups = single_head_groups;
  single.tokens_per_tile = 16 / single_heads_per_tile;
  single.single_tokens = 1;
  single.seg_keys = 0;
  single.num_splits = 1;
  single.plan = plan;
  single.items_grid = items_grid;
  single.qkv = static_cast<const bf16_t*>(qkv);
  single.q_weight = q_weight;
  single.k_weight = k_weight;
  single.rope_table = rope_table;
  single.table_positions = table_positions;
  single.eps = eps;
  portion.partial = nullptr;
  portion.seq_first = portion_first;
  portion.seq_count = portion_count;
  portion.tiles = portion_tiles;
  portion.heads_per_tile = portion_heads_per_tile;
  portion.head_groups = portion_head_groups;
  portion.tokens_per_tile = portion_tokens_per_tile;
  portion.single_tokens = 0;
  portion.seg_keys = 0;
  portion.num_splits = 1;
  portion.plan = nullptr;
  portion.items_grid = 0;
  portion.qkv = nullptr;
  portion.q_weight = nullptr;
  portion.k_weight = nullptr;
  portion.rope_table = nullptr;
  portion.table_positions = 0;
  portion.eps = 0.f;
  portion.units = units_of_device();
  if (portion.units == 0) return -3;
  return launch_pair(single, portion, portion_tiles, stream);
}
