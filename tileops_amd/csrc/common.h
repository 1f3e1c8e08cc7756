// Shared host/device declarations for the gfx950 paged GQA decode library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mi355_tileops.h"

namespace mi355 {

// Measurement aid, OR-ed into the kernel selector of the decode entry points by this package's own benchmark: launch the
// attention kernel only and leave the partial results in the workspace unmerged (the output is then incomplete), so
// that the dominant kernel can be timed alone.  Not part of the public interface.
constexpr int kKernelFlagSkipCombine = 0x100;

constexpr float kLog2e = 1.4426950408889634f;
// Finite stand-in for "-infinity" as the running maximum: exp2(-inf - kNegFloor) == 0 and
// exp2(kNegFloor - kNegFloor) == 1, so empty tiles and empty splits never produce NaN.
constexpr float kNegFloor = -1.0e30f;

// Everything one decode call needs, passed to the kernels by value.
struct DecodeParams {
  const void* q;
  const void* k;
  const void* v;
  const float* k_scale;
  const float* v_scale;
  const int32_t* seqlens;
  const int32_t* block_table;
  int64_t bt_row_stride;
  // Contiguous cache (no block table): block_table and seqlens are null, sequence b occupies tokens
  // [b*contig_stride, b*contig_stride + uniform_len) of k/v, and page_size is only the tile granule.
  int64_t contig_stride;
  int uniform_len;
  // Packed variable-length queries (prefill chunks): q and out are [total_q, heads, dim], sequence b owns query rows
  // [cu_q[b], cu_q[b+1]); q_len is then the largest chunk.  Null = every sequence has q_len query tokens.
  const int32_t* cu_q;
  int len_excludes_new;  // with cu_q: seqlens[b] counts the context *before* the chunk; the chunk's tokens are added
  // Packed contiguous keys/values (the chunk's own tokens): sequence b occupies tokens [kv_starts[b], ...) of k/v.
  const int32_t* kv_starts;
  int scale_per_tensor;  // fp8: k_scale/v_scale hold one value each instead of one per (token, kv head)
  // When set, the result leaves as fp32 rows plus log2-domain log-sum-exp ([total_q, heads, dim] / [total_q, heads])
  // instead of 16-bit rows in out, so that two calls over disjoint key sets can be merged afterwards.
  float* final_o;
  float* final_lse;
  // MFMA kernel: when set, every query row starts from this earlier result over a disjoint key set (fp32 rows and
  // log2-domain log-sum-exp as written through final_o / final_lse) instead of from nothing, so the call's output is
  // already the merge of both.
  const float* init_o;
  const float* init_lse;
  void* out;
  float* part_o;    // workspace: normalised partial outputs, fp32 (or rows of the query's 16-bit type: part16)
  float* part_lse;  // workspace: log2-domain log-sum-exp per partial (-inf = empty)
  int batch, q_len, heads, heads_kv, dim, page_size;
  int group;        // heads / heads_kv
  int rows;         // q_len * group : query rows that share one kv head
  int64_t n_pages;  // n_phys_tokens / page_size
  int max_len;      // tokens one block-table row (or one sequence's slot of a contiguous cache) can address: lengths are clamped to it
  float score_scale;  // sm_scale (softcap on) or sm_scale * log2e (softcap off)
  float softcap;      // 0 = off
  float cap_log2e;    // softcap * log2e
  float inv_cap_scale;  // sm_scale / softcap
  int negate_q;         // MFMA kernel: flip the sign of the query (set by its launcher for a negative scale)
  int causal;
  // generic kernel: fixed-length KV splits per sequence
  int max_splits;
  int split_tokens;
  // MFMA kernel: even partition of the KV tile stream
  int n_parts;
  int part16;        // partial output rows are stored in the query's 16-bit type (the dtype of the reference's partials)
};

// Context length of sequence b: per-sequence array (paged cache) or one value for all (contiguous cache), clamped to
// [0, max_len] so that a corrupt length can neither run the kernels past the sequence's block-table row nor make the
// tile-stream sums negative.
__device__ __forceinline__ int q_len_of(const DecodeParams& p, int b) { return p.cu_q ? p.cu_q[b + 1] - p.cu_q[b] : p.q_len; }
__device__ __forceinline__ int64_t q_row0_of(const DecodeParams& p, int b) { return p.cu_q ? (int64_t)p.cu_q[b] : (int64_t)b * p.q_len; }
// kLand (per-lane callers inside loops that keep direct-to-LDS loads in flight): an empty asm reads the loaded registers
// right after the loads, so the wait for them stands here.  Otherwise the clamp and its wait sink into the branch that
// has query rows, the other branch leaves the load formally outstanding, and the compiler protects the next write of
// that register -- wherever it is, in practice an LDS read of the tile loop -- with a vmcnt(0) that drains every
// prefetch on every tile (measured: 146 -> 167 us on the eight-query-token FP8 workload).
// The two loads of a length, apart from what is made of them, so that a caller can request them early and use them late.
struct RawSeqLen {
  int len, ql;
};
__device__ __forceinline__ RawSeqLen seq_len_load(const DecodeParams& p, int b) {
  RawSeqLen r;
  r.len = p.seqlens ? p.seqlens[b] : p.uniform_len;
  r.ql = 1;
  if (p.cu_q) r.ql = p.cu_q[b + 1] - p.cu_q[b];
  return r;
}
__device__ __forceinline__ int seq_len_finish(const DecodeParams& p, RawSeqLen r) {
  int len = r.len;
  if (p.cu_q) {
    if (r.ql <= 0) return 0;  // no query rows: nothing to compute, the sequence contributes no tile
    // (saturating: a corrupt length near INT_MAX must end up clamped to max_len, not wrapped to a negative number)
    if (p.len_excludes_new) len = len > p.max_len - r.ql ? p.max_len : len + r.ql;
  }
  return min(max(len, 0), p.max_len);
}
template <bool kLand = false>
__device__ __forceinline__ int seq_len_of(const DecodeParams& p, int b) {
  RawSeqLen r = seq_len_load(p, b);
  if constexpr (kLand) asm volatile("" : "+v"(r.len), "+v"(r.ql));
  return seq_len_finish(p, r);
}

// Number of KV splits of one sequence and the (tile-aligned) tokens per split, generic kernel.
// Used identically by the attention kernel and its combine kernel.
__host__ __device__ inline void split_geometry(int len, int split_tokens, int max_splits, int* n_splits, int* chunk) {
  int n = (len + split_tokens - 1) / split_tokens;
  if (n > max_splits) n = max_splits;
  if (n < 1) n = 1;
  int c = (len + n - 1) / n;
  c = (c + 63) / 64 * 64;
  if (c < 64) c = 64;
  *chunk = c;
  *n_splits = len > 0 ? (len + c - 1) / c : 1;
}

// --- launchers (defined in the kernel translation units) -----------------------------------------
const char* launch_generic(const DecodeParams& p, int q_dtype, int kv_dtype, hipStream_t s);
const char* launch_generic_combine(const DecodeParams& p, int q_dtype, hipStream_t s);
bool mfma_supported(int q_len, int heads, int heads_kv, int dim, int page_size, int q_dtype, int kv_dtype, float softcap);
int mfma_num_parts(int heads_kv, int rows, int dim, int kv_dtype, int compute_units);
size_t mfma_workspace_bytes(int n_parts, int heads_kv, int rows, int dim, int batch);
const char* launch_mfma(const DecodeParams& p, int q_dtype, int kv_dtype, bool skip_combine, hipStream_t s);
// Compute units of the current device (256 on MI355X; that figure also when no device is visible).  Asked once per
// device, and only by entry points that launch: workspace queries plan for 256 and touch no device.
int device_cu_count();
const char* launch_gather_probe(const void* cache, const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride,
                                void* dense_out, int batch, int64_t max_len, int64_t row_bytes, int page_size,
                                int64_t n_pages, hipStream_t s);
const char* launch_kv_append_chunk(const void* k_new, const void* v_new, void* k_pages, void* v_pages, const float* k_scale,
                                   const float* v_scale, const int32_t* cu_q, const int32_t* cache_seqlens,
                                   const int32_t* block_table, int64_t bt_row_stride, int batch, int64_t total_q, int heads_kv,
                                   int dim, int page_size, int64_t n_pages, int x_dtype, int cache_dtype, hipStream_t s);
const char* launch_rope_append_chunk(const void* q, const void* k_new, const void* v_new, void* q_rot, void* k_pages, void* v_pages,
                                     const void* cos_table, const void* sin_table, const int32_t* cu_q,
                                     const int32_t* cache_seqlens, const int32_t* block_table, int64_t bt_row_stride, int batch,
                                     int64_t total_q, int heads, int heads_kv, int dim, int rotary_dim, int64_t max_position,
                                     int page_size, int64_t n_pages, int x_dtype, hipStream_t s);
const char* launch_dequant_pack_chunk(const void* k_pages, const void* v_pages, const void* k_new, const void* v_new,
                                      const float* k_scale, const float* v_scale, const int32_t* cu_q, const int32_t* cache_seqlens,
                                      const int32_t* block_table, int64_t bt_row_stride, void* kp, void* vp, int32_t* kv_starts,
                                      int batch, int heads_kv, int dim, int page_size, int64_t n_pages, int stride, int x_dtype,
                                      hipStream_t s);
const char* launch_merge_two(const float* o_a, const float* lse_a, const float* o_b, const float* lse_b, void* out,
                             int64_t rows, int dim, int q_dtype, hipStream_t s);
const char* launch_prefill_input_facts(const int32_t* cu_q, const int32_t* cache_seqlens, const int32_t* block_table,
                                       int64_t bt_row_stride, const float* k_scale, const float* v_scale, int batch, int max_pages,
                                       int32_t* facts, hipStream_t s);
const char* launch_kv_append_fp8(const void* x_new, void* cache, float* scale, const int32_t* seqlens,
                                 const int32_t* block_table, int64_t bt_row_stride, int batch, int heads_kv, int dim,
                                 int page_size, int64_t n_pages, int x_dtype, hipStream_t s);

}  // namespace mi355
