/*
 * mi355_tileops.h -- C ABI of the MI355X (gfx950) paged GQA decode library.
 *
 * Plain pointers and sizes only; every entry point enqueues work on the given HIP stream and returns.
 * No entry point synchronises the device, reads device memory on the host, or allocates device memory:
 * the caller owns inputs, output and workspace.  All functions return 0 on success or a negative
 * MI355_E* code; mi355_last_error() then gives a thread-local message.  Nothing throws or aborts.
 *
 * The reference (tile-ai/TileOPs) has no native ABI: its kernels are TileLang programs JIT-compiled to
 * CUDA and reached through torch custom ops.  Each declaration below cites the reference interface whose
 * job it takes over.
 */
#ifndef MI355_TILEOPS_H
#define MI355_TILEOPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_ABI_VERSION 1

/* element types */
#define MI355_DT_BF16 0
#define MI355_DT_FP16 1
#define MI355_DT_FP8_E4M3FN 2 /* OCP e4m3fn (gfx950 native); KV cache only */

/* kernel selection for mi355_gqa_paged_decode(): which implementation serves the call */
#define MI355_KERNEL_AUTO 0    /* MFMA kernel when the shape qualifies, else the generic one */
#define MI355_KERNEL_GENERIC 1 /* VALU kernel: any head_dim in {64,128,256}, any page size, any group */
#define MI355_KERNEL_MFMA 2    /* MFMA kernel (head_dim 64/128/256, 16-bit or FP8 cache, page size 16 or a multiple of 32);
                                  MI355_EUNSUPPORTED if the shape does not qualify */

/* error codes */
#define MI355_OK 0
#define MI355_EINVAL (-1)       /* an argument violates the contract (message names it) */
#define MI355_EUNSUPPORTED (-2) /* legal call, but no kernel in this library serves it */
#define MI355_EWORKSPACE (-3)   /* workspace pointer missing or too small */
#define MI355_ELAUNCH (-4)      /* HIP reported an error at launch */
#define MI355_EDEVICE (-5)      /* no current HIP device, or it is not gfx950: returned by every entry point that would
                                   launch, before anything is launched (workspace queries touch no device) */

/* Version of this ABI (MI355_ABI_VERSION of the library that was loaded). */
int mi355_abi_version(void);

/* Message for the last error on the calling thread ("" if none). The pointer stays valid until the
 * next failing call on the same thread. */
const char* mi355_last_error(void);

/*
 * Workspace requirement and split plan for one decode call of the given shape.
 *
 * Replaces the host prologue of GQADecodePagedKernel.forward
 * (src/tileops/kernels/attention/gqa_decode_paged.py:683-721), which reads max(real_seqlen_kv) back to
 * the host, builds split_length with torch ops and allocates glse / Output_partial per call.  Here the
 * plan depends only on shapes, so nothing is read back; the per-sequence split bounds are derived from
 * real_seqlen_kv inside the kernels.
 *
 *   max_blocks_per_seq : width of block_table actually usable (>= ceil(max context / page_size))
 *   num_split_in       : 0 = choose; > 0 = upper bound on KV splits per sequence (generic kernel) /
 *                        number of equal ranges the MFMA kernel cuts the KV tile stream into (at most 4096;
 *                        0 = one range per wave the chip holds, which is what measures best -- the knob is
 *                        there for the kernel class's autotuner)
 *   kernel             : MI355_KERNEL_*
 * Outputs: *workspace_bytes (may be 0), *num_split_out (splits per sequence the generic kernel will
 * use at most; number of stream partitions for the MFMA kernel), *kernel_out (the kernel AUTO resolved to).
 * The query touches no device and initialises no HIP runtime: with num_split_in == 0 it plans for the 256 compute
 * units of an MI355X.  A launch on a device with fewer compute units uses fewer partitions and so never needs more
 * workspace than the query reported; pass num_split_out back as num_split to get exactly the plan that was sized.
 */
int mi355_gqa_paged_decode_workspace(int batch, int q_len, int heads, int heads_kv, int dim, int page_size,
                                     int64_t max_blocks_per_seq, int q_dtype, int kv_dtype, int num_split_in,
                                     int kernel, size_t* workspace_bytes, int* num_split_out, int* kernel_out);

/*
 * Paged GQA decode attention, one call = one forward of
 * GroupedQueryAttentionDecodePagedWithKVCacheFwdOp
 * (src/tileops/ops/attention/gqa.py:1443-1454 -> GQADecodePagedKernel.forward,
 *  src/tileops/kernels/attention/gqa_decode_paged.py:669-746; custom-op argument lists :401-421, :451-475),
 * i.e. the reference's no-split kernel (:75-168), split kernel (:209-342) and combine (:344-374).
 *
 *   q            [batch, q_len, heads, dim]  q_dtype (bf16|fp16), contiguous.  q_len == 1 is the reference op.
 *   k, v         [n_phys_tokens, heads_kv, dim]  kv_dtype, contiguous: the physical page pool,
 *                page p = tokens [p*page_size, (p+1)*page_size)
 *   k_scale,
 *   v_scale      [n_phys_tokens, heads_kv] fp32 per-token-per-head dequant scales (x = fp8 * scale);
 *                required iff kv_dtype == MI355_DT_FP8_E4M3FN, else NULL
 *                (format of src/tileops/kernels/fp8_quant.py:44-60; dequant as kernels/attention/gqa_fwd.py:1063-1065)
 *   seqlens      [batch] int32: tokens of context per sequence, INCLUDING the q_len new tokens
 *   block_table  [batch, >= ceil(seqlens[b]/page_size)] int32 physical page ids, row stride bt_row_stride (elements)
 *   out          [batch, q_len, heads, dim] q_dtype
 *   workspace    >= the size mi355_gqa_paged_decode_workspace() reports for the same arguments, 256-byte aligned.
 *                It holds what the reference keeps in glse / Output_partial (gqa_decode_paged.py:718-722): log-sum-exps in
 *                fp32; partial output rows in fp32, or -- on the MFMA kernel, with q_len > 1 and more than 4096 query
 *                rows (batch * q_len * heads) -- in q_dtype, the type the reference gives every partial (:216-217)
 *   sm_scale     softmax scale applied to q.k  (the op passes dim**-0.5 unless overridden, gqa.py:81-82)
 *   softcap      0 = off, else scores := softcap * tanh(scores / softcap)  (online_softmax.py:153-173)
 *   causal       with q_len > 1: query i sees key j iff j <= i + (seqlens[b] - q_len)  (gqa.py:558-562)
 *   num_split    as num_split_in above;  kernel as above
 *
 * Sequences with seqlens[b] == 0 produce zeros.  Tokens not addressed by (block_table, seqlens) are never read.
 * Lengths are clamped on the device to [0, bt_row_stride * page_size], what one block-table row can address, so a
 * corrupt seqlens[b] cannot make a kernel read the table past the sequence's row; page ids are clamped into the pool.
 */
int mi355_gqa_paged_decode(const void* q, const void* k, const void* v, const float* k_scale,
                           const float* v_scale, const int32_t* seqlens, const int32_t* block_table,
                           int64_t bt_row_stride, void* out, void* workspace, size_t workspace_bytes, int batch,
                           int q_len, int heads, int heads_kv, int dim, int page_size, int64_t n_phys_tokens,
                           int q_dtype, int kv_dtype, float sm_scale, float softcap, int causal, int num_split,
                           int kernel, void* hip_stream);

/*
 * mi355_gqa_paged_decode() for callers that cannot allocate: the same call, with the library's own scratch in place of the
 * workspace argument.  It has no counterpart in the reference (whose forward allocates glse / Output_partial with torch on
 * every call, gqa_decode_paged.py:718-721); it is for callers that cannot call hipMalloc or hold a workspace -- code under
 * HIP graph capture, tight serving loops, harnesses that forbid allocation.  It calls no hipMalloc / hipFree or other
 * allocating routine; the scratch is an 80 MiB array in the library's device image, one per GPU, held until the process ends.
 * Limits: calls whose workspace requirement (mi355_gqa_paged_decode_workspace) exceeds 80 MiB are refused with
 * MI355_EWORKSPACE and a message (every plan of the MFMA kernel fits: at most 67.6 MB whatever the shape; the general
 * kernel's plan grows with batch x splits and may not);
 * all calls on one GPU share that GPU's array, so two calls that overlap in time on one GPU (different streams) race --
 * keep such calls on one stream, or use mi355_gqa_paged_decode with separate workspaces.  Arguments as there.
 * Under graph capture: the first call on a device (of a process, per kernel instance it selects) does one-time set-up
 * that is not stream work -- it asks the runtime for the array's device address and raises the kernels' LDS limit -- and
 * must not itself be captured.  Make one ordinary call of the same shape on that device first, then capture; captured
 * calls enqueue the two kernels and nothing else (no memset node), and replays pick up changed cache contents, lengths
 * and block tables in place.
 * Cost: the array is part of the library's device image, so every process that loads the library holds 80 MiB on every
 * GPU it initialises, whether or not it ever calls this entry point (16 processes on one GPU: 1.3 GB).
 */
int mi355_gqa_paged_decode_static(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                  const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride, void* out,
                                  int batch, int q_len, int heads, int heads_kv, int dim, int page_size,
                                  int64_t n_phys_tokens, int q_dtype, int kv_dtype, float sm_scale, float softcap, int causal,
                                  int num_split, int kernel, void* hip_stream);

/*
 * GQA decode over a contiguous (un-paged) KV cache: one call = one forward of
 * GroupedQueryAttentionDecodeWithKVCacheFwdOp (src/tileops/ops/attention/gqa.py:1336-1350 ->
 * GQADecodeKernel.forward, src/tileops/kernels/attention/gqa_decode.py:555-612; custom-op argument lists
 * :312-335, :358-385), i.e. the reference's no-split kernel (:24-122), split kernel (:124-310) and its combine.
 * Same kernels as the paged entry point with identity addressing: sequence b occupies tokens
 * [b*kv_seq_stride, b*kv_seq_stride + real_seqlen_kv) of k and v.
 *
 *   q              [batch, q_len, heads, dim]  q_dtype, contiguous (q_len == 1 is the reference op)
 *   k, v           [batch, kv_seq_stride, heads_kv, dim]  kv_dtype, contiguous; only the first real_seqlen_kv tokens
 *                  of each sequence are read, so no zero padding up to a compiled-in length is needed
 *                  (the reference pads to seqlen_kv, gqa.py:1338-1345)
 *   k_scale,
 *   v_scale        [batch, kv_seq_stride, heads_kv] fp32, iff kv_dtype == MI355_DT_FP8_E4M3FN (this library's extension)
 *   real_seqlen_kv tokens of context of every sequence (one value, as in the reference's forward)
 *   workspace      >= what mi355_gqa_decode_workspace() reports for max_seqlen_kv >= real_seqlen_kv
 * The remaining arguments are those of mi355_gqa_paged_decode().
 */
int mi355_gqa_decode_workspace(int batch, int q_len, int heads, int heads_kv, int dim, int64_t max_seqlen_kv, int q_dtype,
                               int kv_dtype, int num_split_in, int kernel, size_t* workspace_bytes, int* num_split_out,
                               int* kernel_out);
int mi355_gqa_decode(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale, void* out,
                     void* workspace, size_t workspace_bytes, int batch, int q_len, int heads, int heads_kv, int dim,
                     int64_t kv_seq_stride, int real_seqlen_kv, int q_dtype, int kv_dtype, float sm_scale, float softcap,
                     int causal, int num_split, int kernel, void* hip_stream);

/*
 * Packed GQA prefill chunk with paged KV-cache append: one call = one forward of
 * GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp (src/tileops/ops/attention/gqa.py:1072-1140 ->
 * GQAPrefillPagedWithKVCacheFwdKernel / GQAPrefillPagedWithFP8KVCacheFwdKernel,
 * src/tileops/kernels/attention/gqa_fwd.py:600-1000 and :1005-1460).  The third reference kernel, fused RoPE, is
 * mi355_gqa_prefill_paged_rope() below.
 *
 *   q              [total_q, heads, dim] q_dtype: the chunks of all sequences packed; sequence b owns rows
 *                  [cu_seqlens_q[b], cu_seqlens_q[b+1])
 *   k_new, v_new   [total_q, heads_kv, dim] q_dtype: keys/values of the same rows
 *   k_pages,
 *   v_pages        [n_phys_tokens, heads_kv, dim] cache_dtype (q_dtype or fp8): the page pool.  The chunk is appended at
 *                  logical positions cache_seqlens[b] + i (16-bit: copied; fp8: clamp(x / scale, +-448) -> e4m3fn,
 *                  gqa_fwd.py:1059-1061, :1124-1168)
 *   k_scale,
 *   v_scale        [1] fp32 per-tensor dequantisation scales (x = fp8 * scale); read only with an fp8 cache
 *   cu_seqlens_q   [batch + 1] int32;  cache_seqlens [batch] int32: context length of each sequence before the append
 *   block_table    [batch, >= ceil((cache_seqlens[b] + q_len_b) / page_size)] int32, row stride bt_row_stride
 *   out            [total_q, heads, dim] q_dtype
 *   max_seqlen_q   upper bound of the chunk lengths (sizes the launch; a longer chunk would lose its last rows)
 *   causal         query i of a chunk sees the old tokens and chunk tokens j <= i (gqa_fwd.py:1247-1256); 0: all of them
 * Attention runs over the dequantised old tokens and the *unquantised* chunk (as the reference: :1180-1245).  With an fp8
 * cache that is either two passes (the fp8 pages, then k_new/v_new, merged by log-sum-exp) or, from 1024 query rows per
 * kv head (max_seqlen_q * heads / heads_kv) on the MFMA kernel, one pass over rows dequantised once into the workspace
 * as (fp8 * scale) rounded to q_dtype (the reference's own dequantisation, :1063-1065) with the chunk behind them.  The
 * second form needs 4 * batch * max_pages_per_req * page_size * heads_kv * dim bytes of workspace and is only taken up
 * to 4 GiB of it; the workspace query answers for whichever form the same arguments select.
 * Sequences with an empty chunk produce no output rows and append nothing.  A chunk token whose position
 * cache_seqlens[b] + i the block-table row cannot address (negative, or page index >= bt_row_stride) is not appended.
 */
int mi355_gqa_prefill_paged_workspace(int batch, int max_seqlen_q, int64_t total_q, int heads, int heads_kv, int dim,
                                      int page_size, int64_t max_pages_per_req, int q_dtype, int cache_dtype, int kernel,
                                      size_t* workspace_bytes);
int mi355_gqa_prefill_paged(const void* q, const void* k_new, const void* v_new, void* k_pages, void* v_pages,
                            const float* k_scale, const float* v_scale, const int32_t* cu_seqlens_q,
                            const int32_t* cache_seqlens, const int32_t* block_table, int64_t bt_row_stride, void* out,
                            void* workspace, size_t workspace_bytes, int batch, int max_seqlen_q, int64_t total_q, int heads,
                            int heads_kv, int dim, int page_size, int64_t n_phys_tokens, int q_dtype, int cache_dtype,
                            float sm_scale, float softcap, int causal, int kernel, void* hip_stream);

/*
 * The same prefill chunk with rotary position embedding fused in (GPT-NeoX halves), 16-bit cache only.  Replaces
 * GQAPrefillPagedWithKVCacheRopeFwdKernel.forward and its two TileLang kernels
 * (src/tileops/kernels/attention/gqa_fwd.py:1464-1582 append, :1660-1917 attention, :2020-2090 class); op side
 * src/tileops/ops/attention/gqa.py:787-823, :891-895, :1048-1065, :1113-1143.
 * Query and new key rows of token t of sequence b are rotated at logical position cache_seqlens[b] + (t - cu_q[b]):
 *   y[d] = x[d]*cos[pos][d % half] + r*sin[pos][d % half],  half = rotary_dim / 2,
 *   r = -x[d + half] for d < half, +x[d - half] for half <= d < rotary_dim;  y[d] = x[d] for d >= rotary_dim
 * (gqa_fwd.py:1521-1535, :1755-1768), products in fp32, rounded once to q_dtype.  The rotated keys go into the pages
 * (values are copied), the rotated queries into the workspace, and attention runs as in mi355_gqa_prefill_paged.
 *   cos_table,
 *   sin_table      [max_position, rotary_dim / 2] q_dtype (src/tileops/ops/rope.py:97-120)
 *   rotary_dim     even, 0 < rotary_dim <= dim
 *   max_position   rows of the tables; the caller guarantees cache_seqlens[b] + q_len_b <= max_position
 *                  (gqa.py:1032-1036); positions beyond are clamped to the last row rather than read out of bounds
 * q, k_new and v_new are not modified.
 */
int mi355_gqa_prefill_paged_rope_workspace(int batch, int max_seqlen_q, int64_t total_q, int heads, int heads_kv, int dim,
                                           int page_size, int64_t max_pages_per_req, int q_dtype, int kernel,
                                           size_t* workspace_bytes);
int mi355_gqa_prefill_paged_rope(const void* q, const void* k_new, const void* v_new, void* k_pages, void* v_pages,
                                 const void* cos_table, const void* sin_table, const int32_t* cu_seqlens_q,
                                 const int32_t* cache_seqlens, const int32_t* block_table, int64_t bt_row_stride, void* out,
                                 void* workspace, size_t workspace_bytes, int batch, int max_seqlen_q, int64_t total_q,
                                 int heads, int heads_kv, int dim, int page_size, int64_t n_phys_tokens, int q_dtype,
                                 int rotary_dim, int64_t max_position, float sm_scale, float softcap, int causal, int kernel,
                                 void* hip_stream);

/*
 * Index-probe: materialise the logical KV rows a decode call would read, with the same device page
 * arithmetic the attention kernels use.  dense_out [batch, max_len, heads_kv * dim] elem_bytes-wide
 * elements; rows t >= seqlens[b] are left untouched.  Lets a test compare the gather bit-for-bit with
 * k.view(P, page, H_kv, D)[block_table[b, :n]] -- the page reassembly of the reference's ref_program
 * (tests/ops/attention/test_gqa_decode_paged.py:46-59).
 */
int mi355_gather_probe(const void* cache, const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride,
                       void* dense_out, int batch, int64_t max_len, int64_t row_bytes, int page_size,
                       int64_t n_phys_tokens, void* hip_stream);

/*
 * Append one new token per sequence to a paged FP8 cache: per-(token, kv-head) absmax/448 scale,
 * clamp(x/scale, +-448) -> e4m3fn (round-to-nearest-even), written at logical position seqlens[b]-1.
 * Takes over the per-token quantizer FP8QuantKernel (src/tileops/kernels/fp8_quant.py:14-64) fused with
 * the page append of the paged prefill kernel (src/tileops/kernels/attention/gqa_fwd.py:1124-1168).
 *   x_new [batch, heads_kv, dim] x_dtype (bf16|fp16); cache [n_phys_tokens, heads_kv, dim] fp8;
 *   scale [n_phys_tokens, heads_kv] fp32.
 */
int mi355_kv_append_fp8(const void* x_new, void* cache, float* scale, const int32_t* seqlens,
                        const int32_t* block_table, int64_t bt_row_stride, int batch, int heads_kv, int dim,
                        int page_size, int64_t n_phys_tokens, int x_dtype, void* hip_stream);

/*
 * The facts behind the value checks that the reference's paged prefill op makes on the host before it launches
 * (GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp._validate_forward_inputs, src/tileops/ops/attention/gqa.py:997-1040:
 * each there a device-to-host read of its own), reduced by one small kernel into ten int32 so that a caller reads them
 * in one transfer (facts: device memory, or pinned host memory, which the kernel writes directly and the caller reads after
 * waiting for the stream):
 *   facts[0], facts[1]  k_scale[0], v_scale[0] finite and positive (1/0; a null scale pointer counts as good)
 *   facts[2] cu_seqlens_q[0]           facts[3] min q_len     facts[4] cu_seqlens_q[batch]   facts[5] max q_len
 *   facts[6] min cache_seqlens         facts[7] max (cache_seqlens + q_len), saturated to int32
 *   facts[8], facts[9]  min and max block_table entry over the batch x max_pages_per_req entries
 * Nothing is judged here: which values are errors, and their messages, stay with the caller.
 */
int mi355_prefill_input_facts(const int32_t* cu_seqlens_q, const int32_t* cache_seqlens, const int32_t* block_table,
                              int64_t bt_row_stride, const float* k_scale, const float* v_scale, int batch,
                              int max_pages_per_req, int32_t* facts, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_TILEOPS_H */
