// C entry points of the kernel library.  Every function enqueues on `stream` and returns 0, a hipError_t of the
// launch, -1 for an unknown dtype code, -2 for sizes the kernel does not take or -3 for sizes beyond a fixed buffer.  dtype codes: 0 float32,
// 1 bfloat16.  Pointers are device pointers; shapes are checked by the caller on the host.
#pragma once

#include <hip/hip_runtime.h>

extern "C" {

int akv_embed(const int* ids, const void* table, int table_dtype, float* out, int tokens, int hidden, int vocab,
              const int* seq_of_token, const int* seq_slots, const int* slot_words, hipStream_t stream);
// out[0..7]: words per slot and the indices of its named words, as the kernels were compiled (see common.h)
int akv_slot_layout(int* out);
int akv_step_prologue(int* state, long state_size, const int* patches, const int* count, int capacity,
                      const int* seq_slots, const int* seq_lens, int seqs, hipStream_t stream);
int akv_add_rmsnorm(float* stream_buf, const void* delta, const float* weight, float eps, void* out, int dtype,
                    int tokens, int hidden, hipStream_t stream);
int akv_rmsnorm_rows(const void* x, long token_stride, const float* weight, float eps, void* out, int dtype,
                     long tokens, int heads, int width, hipStream_t stream);
int akv_copy_rows(const void* x, long token_stride, void* out, int dtype, long tokens, int heads, int width,
                  hipStream_t stream);
int akv_gather_rows(const float* stream_buf, const void* pending, int dtype, const int* rows, float* out, int wanted,
                    int hidden, int tokens, hipStream_t stream);
int akv_swiglu(const void* gate_up, void* out, int dtype, long tokens, int inter, hipStream_t stream);
// Reads `bytes` (a multiple of 16) once, as the decode products read their weights, and leaves the xor of the words a
// block read in out[block]: a measure of what memory gives to a kernel that does nothing else.
int akv_read_probe(const void* data, long bytes, unsigned int* out, int blocks, hipStream_t stream);
int akv_rope_table(const float* inv_freq, float* table, int positions, int half, hipStream_t stream);
int akv_rope(void* x, int dtype, const int* positions, const float* table, long tokens, int heads, int dim,
             int table_positions, hipStream_t stream);
int akv_kv_write(const void* k, long k_stride, const void* v, long v_stride, const int* slot_map, void* k_pages,
                 void* v_pages, int dtype, long tokens, int kv_heads, int dim, int page_size, long num_pages,
                 hipStream_t stream);
int akv_qk_norm_rope_write(const void* qkv, const float* q_weight, const float* k_weight, float eps,
                           const float* table, int table_positions, const int* positions, const int* slot_map,
                           void* k_pages, void* v_pages, void* q_out, int dtype, long tokens, int q_heads,
                           int kv_heads, int dim, int page_size, long num_pages, hipStream_t stream);
// Products y = x W^T (+ bias): `bias` [outs] float32 or null, added to the float32 sums before they are rounded.
int akv_linear_tiled(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype, int rows, int outs,
                     int k, const float* bias, hipStream_t stream);
int akv_linear_packed(const void* x, const void* wp, void* y, int y_dtype, int rows, int outs, int k, int n_tiles,
                      int k_tiles, int x_packed, const float* bias, hipStream_t stream);
int akv_linear_packed_swiglu(const void* x, const void* wp, void* y, int y_dtype, int rows, int inter, int k,
                             int n_tiles, int k_tiles, int x_packed, hipStream_t stream);
int akv_linear_packed_normed(const float* stream_in, const void* delta, const float* norm_weight, float eps,
                             float* stream_out, const void* wp, void* y, int rows, int outs, int k, int n_tiles,
                             int k_tiles, int gated, const float* bias, hipStream_t stream);
int akv_pack_rows(const void* x, void* xp, int rows, int k, hipStream_t stream);
// No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc): akv_pack_rows + akv_linear_packed(x_packed = 1) as one call
// that allocates nothing - the repacked activations live in 4 MiB of static device memory that each GPU holds from
// the library's load to the end of the process.  Up to 64 rows with ceil(rows / 16) * 16 * k <= 2,097,152 elements;
// -3 beyond that.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
// threads) race; calls that follow each other on a stream do not.
int akv_linear_packed_static(const void* x, const void* wp, void* y, int y_dtype, int rows, int outs, int k,
                             int n_tiles, int k_tiles, hipStream_t stream);
int akv_linear_decode_plan(int rt, int n_tiles, int k_tiles, int k, int normed_rows, int may_straddle, int* out);
int akv_linear_adds(const void* x, const void* wp, float* stream_out, float* sums_out, float* pieces,
                    unsigned int* arrivals, int exchange_tiles, int rows, int outs, int k, int n_tiles, int k_tiles,
                    const float* bias, hipStream_t stream);
int akv_linear_scaled(const float* stream_in, const float* sums, int sum_tiles, const float* gain, float eps,
                      const void* wp, void* y, float* pieces, unsigned int* arrivals, int exchange_tiles, int rows,
                      int outs, int k, int n_tiles, int k_tiles, int gated, int row_tiles, const float* bias,
                      hipStream_t stream);
int akv_linear_adds_rows(const void* x, const void* wp, float* stream_out, float* sums_out, float* pieces,
                         unsigned int* arrivals, int exchange_tiles, int rows, int outs, int k, int n_tiles, int k_tiles,
                         const float* bias, void* rows_out, const float* gain, hipStream_t stream);
int akv_linear_rowscaled(const void* x, const float* sums, int sum_tiles, float eps, const void* wp, void* y,
                         float* pieces, unsigned int* arrivals, int exchange_tiles, int rows, int outs, int k,
                         int n_tiles, int k_tiles, int gated, int row_tiles, const float* bias, hipStream_t stream);
}
