// Page-table utilities for gfx950: the index-probe gather and the FP8 KV-cache append.
#include <climits>
#include "common.h"
#include "device_utils.h"

namespace mi355 {

// One workgroup per (logical token, sequence): copy the physical row the block table names into the
// dense [batch, max_len, row_bytes] output.  Uses physical_token(), the page arithmetic of the generic attention
// kernel and of the append kernels below, so a bit-exact comparison against torch indexing pins that arithmetic.
// (The MFMA attention kernel walks the table with its own incremental cursor; its gather is pinned bit-exactly by a
// test that makes one key dominant and reads the physical row id back out of the attention output.)
__global__ void gather_probe_kernel(const uint32_t* __restrict__ cache, const int32_t* __restrict__ seqlens,
                                    const int32_t* __restrict__ block_table, int64_t bt_row_stride,
                                    uint32_t* __restrict__ dense_out, int64_t max_len, int64_t row_dwords,
                                    int page_size, int64_t n_pages) {
  const int b = blockIdx.y;
  const int64_t cap = bt_row_stride * (int64_t)page_size;  // what the sequence's block-table row can address
  const int64_t len = seqlens[b] < cap ? seqlens[b] : cap;
  for (int64_t t = blockIdx.x; t < len && t < max_len; t += gridDim.x) {
    const int64_t phys = physical_token(block_table + (int64_t)b * bt_row_stride, (int)t, page_size, n_pages);
    const uint32_t* src = cache + phys * row_dwords;
    uint32_t* dst = dense_out + ((int64_t)b * max_len + t) * row_dwords;
    for (int64_t i = threadIdx.x; i < row_dwords; i += blockDim.x) dst[i] = src[i];
  }
}

const char* launch_gather_probe(const void* cache, const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride,
                                void* dense_out, int batch, int64_t max_len, int64_t row_bytes, int page_size,
                                int64_t n_pages, hipStream_t s) {
  if (batch == 0 || max_len == 0) return nullptr;
  int gx = (int)(max_len < 4096 ? max_len : 4096);
  hipLaunchKernelGGL(gather_probe_kernel, dim3(gx, batch), dim3(256), 0, s, (const uint32_t*)cache, seqlens, block_table,
                     bt_row_stride, (uint32_t*)dense_out, max_len, row_bytes / 4, page_size, n_pages);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

// One wave per (sequence, kv head): absmax over the head vector, scale = max(absmax, 1e-4) / 448,
// q = e4m3fn(clamp(x / scale, -448, 448)), stored at the sequence's last logical position.
template <typename XT>
__global__ __launch_bounds__(64) void kv_append_fp8_kernel(const uint16_t* __restrict__ x_new, uint8_t* __restrict__ cache,
                                                           float* __restrict__ scale, const int32_t* __restrict__ seqlens,
                                                           const int32_t* __restrict__ block_table, int64_t bt_row_stride,
                                                           int heads_kv, int dim, int page_size, int64_t n_pages) {
  const int b = blockIdx.y, kvh = blockIdx.x, lane = threadIdx.x;
  const int len = seqlens[b];
  if (len <= 0 || (len - 1) / page_size >= bt_row_stride) return;  // a position the block-table row cannot address: write nothing
  const int64_t phys = physical_token(block_table + (int64_t)b * bt_row_stride, len - 1, page_size, n_pages);
  const uint16_t* xp = x_new + ((int64_t)b * heads_kv + kvh) * dim;
  const int per = dim / 64 > 0 ? dim / 64 : 1;  // dim in {64,128,256}: 1, 2 or 4 elements per lane, consecutive
  float xv[4];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (i < per) {
      uint32_t bits = xp[lane * per + i];
      uint32_t raw[1] = {bits};
      float tmp[2];
      Unpack<XT, 2>::run(raw, tmp);
      xv[i] = tmp[0];
      amax = fmaxf(amax, fabsf(xv[i]));
    }
  }
#pragma unroll
  for (int mask = 1; mask < 64; mask <<= 1) amax = fmaxf(amax, __shfl_xor(amax, mask, 64));
  amax = fmaxf(amax, 1e-4f);
  const float sc = amax / 448.0f;
  const int64_t row = phys * heads_kv + kvh;
  if (lane == 0) scale[row] = sc;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (i < per) {
      float t = fminf(fmaxf(xv[i] / sc, -448.0f), 448.0f);
      uint32_t packed = __builtin_amdgcn_cvt_pk_fp8_f32(t, t, 0u, false);  // round-to-nearest-even
      cache[row * dim + lane * per + i] = (uint8_t)(packed & 0xff);
    }
  }
}

const char* launch_kv_append_fp8(const void* x_new, void* cache, float* scale, const int32_t* seqlens,
                                 const int32_t* block_table, int64_t bt_row_stride, int batch, int heads_kv, int dim,
                                 int page_size, int64_t n_pages, int x_dtype, hipStream_t s) {
  if (batch == 0) return nullptr;
  dim3 grid(heads_kv, batch);
  if (x_dtype == MI355_DT_BF16)
    hipLaunchKernelGGL(kv_append_fp8_kernel<bf16_tag>, grid, dim3(64), 0, s, (const uint16_t*)x_new, (uint8_t*)cache, scale,
                       seqlens, block_table, bt_row_stride, heads_kv, dim, page_size, n_pages);
  else
    hipLaunchKernelGGL(kv_append_fp8_kernel<fp16_tag>, grid, dim3(64), 0, s, (const uint16_t*)x_new, (uint8_t*)cache, scale,
                       seqlens, block_table, bt_row_stride, heads_kv, dim, page_size, n_pages);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

// The facts behind the value checks of the reference's paged prefill op (src/tileops/ops/attention/gqa.py:997-1040),
// reduced on the device so that the host reads them in one transfer instead of one per check:
//   facts[0] k_scale finite and positive (1/0)      facts[1] v_scale finite and positive (1/0)
//   facts[2] cu_q[0]                                 facts[3] min over b of cu_q[b+1] - cu_q[b]
//   facts[4] cu_q[batch]                             facts[5] max over b of cu_q[b+1] - cu_q[b]
//   facts[6] min cache_seqlens                       facts[7] max over b of cache_seqlens[b] + q_len[b]   (64-bit sums, saturated)
//   facts[8] min block_table entry                   facts[9] max block_table entry
// The block table (batch x max_pages entries, rows bt_row_stride apart) is the bulk of the reading.
__global__ __launch_bounds__(1024) void prefill_input_facts_kernel(const int32_t* __restrict__ cu_q, const int32_t* __restrict__ cache_seqlens,
                                                                   const int32_t* __restrict__ block_table, int64_t bt_row_stride,
                                                                   const float* __restrict__ k_scale, const float* __restrict__ v_scale,
                                                                   int batch, int max_pages, int32_t* __restrict__ facts) {
  // One workgroup of sixteen waves (the ten facts are global minima and maxima: several workgroups would need a second
  // launch or initialised memory to meet in).  A wave takes whole block-table rows, 16 bytes per lane and four such loads
  // in flight when the rows allow it, so that a table of a few thousand entries is one round trip and no index is divided.
  __shared__ int red[6][16];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  int min_q = INT_MAX, max_q = INT_MIN, min_c = INT_MAX, max_tot = INT_MIN, min_p = INT_MAX, max_p = INT_MIN;
  for (int b = t; b < batch; b += 1024) {
    const int ql = cu_q[b + 1] - cu_q[b], c = cache_seqlens[b];
    const int64_t tot = (int64_t)c + ql;
    min_q = min(min_q, ql);
    max_q = max(max_q, ql);
    min_c = min(min_c, c);
    max_tot = max(max_tot, (int)min(max(tot, (int64_t)INT_MIN), (int64_t)INT_MAX));
  }
  const bool vec_ok = (bt_row_stride & 3) == 0 && ((uintptr_t)block_table & 15) == 0;
  const int n_vec = vec_ok ? max_pages >> 2 : 0;  // whole 16-byte groups of a row
  for (int b = wave; b < batch; b += 16) {
    const int32_t* row = block_table + (int64_t)b * bt_row_stride;
    for (int j0 = 0; j0 < n_vec; j0 += 256) {
      int4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int j = j0 + 64 * u + lane;
        v[u] = ((const int4*)row)[j < n_vec ? j : n_vec - 1];  // (past the end: the last group again)
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        min_p = min(min(min_p, v[u].x), min(v[u].y, min(v[u].z, v[u].w)));
        max_p = max(max(max_p, v[u].x), max(v[u].y, max(v[u].z, v[u].w)));
      }
    }
    for (int j = 4 * n_vec + lane; j < max_pages; j += 64) {
      const int v = row[j];
      min_p = min(min_p, v);
      max_p = max(max_p, v);
    }
  }
  int vals[6] = {min_q, max_q, min_c, max_tot, min_p, max_p};
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
#pragma unroll
    for (int f = 0; f < 6; f++) {
      const int o = __shfl_xor(vals[f], m, 64);
      vals[f] = (f & 1) ? max(vals[f], o) : min(vals[f], o);  // facts 0, 2, 4 are minima, 1, 3, 5 maxima
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int f = 0; f < 6; f++) red[f][wave] = vals[f];
  }
  __syncthreads();
  if (t == 0) {
#pragma unroll
    for (int f = 0; f < 6; f++) {
      int r = red[f][0];
      for (int w = 1; w < 16; w++) r = (f & 1) ? max(r, red[f][w]) : min(r, red[f][w]);
      vals[f] = r;
    }
    const float ks = k_scale ? k_scale[0] : 1.f, vs = v_scale ? v_scale[0] : 1.f;
    facts[0] = (isfinite(ks) && ks > 0.f) ? 1 : 0;
    facts[1] = (isfinite(vs) && vs > 0.f) ? 1 : 0;
    facts[2] = cu_q[0];
    facts[3] = vals[0];
    facts[4] = cu_q[batch];
    facts[5] = vals[1];
    facts[6] = vals[2];
    facts[7] = vals[3];
    facts[8] = vals[4];
    facts[9] = vals[5];
  }
}

const char* launch_prefill_input_facts(const int32_t* cu_q, const int32_t* cache_seqlens, const int32_t* block_table,
                                       int64_t bt_row_stride, const float* k_scale, const float* v_scale, int batch, int max_pages,
                                       int32_t* facts, hipStream_t s) {
  hipLaunchKernelGGL(prefill_input_facts_kernel, dim3(1), dim3(1024), 0, s, cu_q, cache_seqlens, block_table, bt_row_stride, k_scale,
                     v_scale, batch, max_pages, facts);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

// Append a packed chunk of new tokens to the paged cache: token t of sequence b (t in [cu_q[b], cu_q[b+1])) goes to
// logical position cache_seqlens[b] + (t - cu_q[b]).  16-bit cache: the row is copied.  FP8 cache: per-tensor scale,
// q = e4m3fn(clamp(x / scale, -448, 448)) -- the append of the reference's paged prefill kernels
// (src/tileops/kernels/attention/gqa_fwd.py:1059-1061, :1124-1168).  One workgroup per token, K and V together.
template <typename XT, bool FP8C>
__global__ __launch_bounds__(256) void kv_append_chunk_kernel(const uint16_t* __restrict__ k_new, const uint16_t* __restrict__ v_new,
                                                              void* __restrict__ k_pages, void* __restrict__ v_pages,
                                                              const float* __restrict__ k_scale, const float* __restrict__ v_scale,
                                                              const int32_t* __restrict__ cu_q, const int32_t* __restrict__ cache_seqlens,
                                                              const int32_t* __restrict__ block_table, int64_t bt_row_stride,
                                                              int batch, int64_t row_elems, int page_size, int64_t n_pages) {
  const int64_t t = blockIdx.x;
  int lo = 0, hi = batch;  // the sequence with cu_q[b] <= t < cu_q[b+1] (empty chunks are skipped by the search)
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid;
  }
  const int b = lo;
  if (t >= cu_q[b + 1]) return;
  const int64_t pos64 = (int64_t)cache_seqlens[b] + (t - cu_q[b]);  // (64-bit: a corrupt length near INT_MAX must not wrap)
  if (pos64 < 0 || pos64 / page_size >= bt_row_stride) return;  // a position the block-table row cannot address: write nothing
  const int pos = (int)pos64;
  const int64_t phys = physical_token(block_table + (int64_t)b * bt_row_stride, pos, page_size, n_pages);
  const uint16_t* ks = k_new + t * row_elems;
  const uint16_t* vs = v_new + t * row_elems;
  if (!FP8C) {
    uint16_t* kd = (uint16_t*)k_pages + phys * row_elems;
    uint16_t* vd = (uint16_t*)v_pages + phys * row_elems;
    for (int64_t i = threadIdx.x * 2; i < row_elems; i += 512) {  // head dims are even: two elements per access
      *(uint32_t*)(kd + i) = *(const uint32_t*)(ks + i);
      *(uint32_t*)(vd + i) = *(const uint32_t*)(vs + i);
    }
  } else {
    const float sk = k_scale[0], sv = v_scale[0];
    uint8_t* kd = (uint8_t*)k_pages + phys * row_elems;
    uint8_t* vd = (uint8_t*)v_pages + phys * row_elems;
    for (int64_t i = threadIdx.x * 2; i < row_elems; i += 512) {
      uint32_t kraw[1] = {*(const uint32_t*)(ks + i)}, vraw[1] = {*(const uint32_t*)(vs + i)};
      float kf[2], vf[2];
      Unpack<XT, 2>::run(kraw, kf);
      Unpack<XT, 2>::run(vraw, vf);
      const float k0 = fminf(fmaxf(kf[0] / sk, -448.0f), 448.0f), k1 = fminf(fmaxf(kf[1] / sk, -448.0f), 448.0f);
      const float v0 = fminf(fmaxf(vf[0] / sv, -448.0f), 448.0f), v1 = fminf(fmaxf(vf[1] / sv, -448.0f), 448.0f);
      *(uint16_t*)(kd + i) = (uint16_t)(__builtin_amdgcn_cvt_pk_fp8_f32(k0, k1, 0u, false) & 0xffff);
      *(uint16_t*)(vd + i) = (uint16_t)(__builtin_amdgcn_cvt_pk_fp8_f32(v0, v1, 0u, false) & 0xffff);
    }
  }
}

const char* launch_kv_append_chunk(const void* k_new, const void* v_new, void* k_pages, void* v_pages, const float* k_scale,
                                   const float* v_scale, const int32_t* cu_q, const int32_t* cache_seqlens,
                                   const int32_t* block_table, int64_t bt_row_stride, int batch, int64_t total_q, int heads_kv,
                                   int dim, int page_size, int64_t n_pages, int x_dtype, int cache_dtype, hipStream_t s) {
  if (batch == 0 || total_q == 0) return nullptr;
  const int64_t row_elems = (int64_t)heads_kv * dim;
  const bool fp8 = cache_dtype == MI355_DT_FP8_E4M3FN, bf = x_dtype == MI355_DT_BF16;
#define MI355_LAUNCH_APPEND(XT, F8)                                                                                           \
  hipLaunchKernelGGL((kv_append_chunk_kernel<XT, F8>), dim3((unsigned)total_q), dim3(256), 0, s, (const uint16_t*)k_new,     \
                     (const uint16_t*)v_new, k_pages, v_pages, k_scale, v_scale, cu_q, cache_seqlens, block_table,           \
                     bt_row_stride, batch, row_elems, page_size, n_pages)
  if (fp8 && bf) MI355_LAUNCH_APPEND(bf16_tag, true);
  else if (fp8) MI355_LAUNCH_APPEND(fp16_tag, true);
  else if (bf) MI355_LAUNCH_APPEND(bf16_tag, false);
  else MI355_LAUNCH_APPEND(fp16_tag, false);
#undef MI355_LAUNCH_APPEND
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

// Rotary position embedding (GPT-NeoX halves) fused with the chunk append, 16-bit cache: for token t of sequence b at
// logical position pos = cache_seqlens[b] + (t - cu_q[b]),
//   y[d] = x[d]*cos[pos][d % half] + r*sin[pos][d % half],  r = -x[d + half] (d < half), +x[d - half] (half <= d < rotary_dim),
//   y[d] = x[d] for d >= rotary_dim,
// applied to every query head (written to q_rot) and every key head (written into the pages); V is copied
// (src/tileops/kernels/attention/gqa_fwd.py:1505-1578 for K/V, :1755-1768 for Q; tables [max_position, half] in the
// element type, src/tileops/ops/rope.py:97-120).  The products are formed in fp32 from the 16-bit operands and rounded
// once.  One workgroup per token.
template <typename XT>
__device__ __forceinline__ float elem_to_f32(uint16_t bits) {
  uint32_t raw[1] = {bits};
  float out[2];
  Unpack<XT, 2>::run(raw, out);
  return out[0];
}

template <typename XT>
__global__ __launch_bounds__(256) void rope_append_chunk_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_new,
                                                                const uint16_t* __restrict__ v_new, uint16_t* __restrict__ q_rot,
                                                                uint16_t* __restrict__ k_pages, uint16_t* __restrict__ v_pages,
                                                                const uint16_t* __restrict__ cos_table, const uint16_t* __restrict__ sin_table,
                                                                const int32_t* __restrict__ cu_q, const int32_t* __restrict__ cache_seqlens,
                                                                const int32_t* __restrict__ block_table, int64_t bt_row_stride, int batch,
                                                                int heads, int heads_kv, int dim, int rotary_dim, int64_t max_position,
                                                                int page_size, int64_t n_pages) {
  const int64_t t = blockIdx.x;
  int lo = 0, hi = batch;  // the sequence with cu_q[b] <= t < cu_q[b+1] (empty chunks are skipped by the search)
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid;
  }
  const int b = lo;
  if (t >= cu_q[b + 1]) return;
  const int64_t pos64 = (int64_t)cache_seqlens[b] + (t - cu_q[b]);  // (64-bit: a corrupt length near INT_MAX must not wrap)
  const bool addressable = pos64 >= 0 && pos64 / page_size < bt_row_stride;  // else: rotate the query, append nothing
  const int pos = addressable ? (int)pos64 : 0;
  const int64_t tpos = pos64 < 0 ? 0 : (pos64 < max_position ? pos64 : max_position - 1);  // the caller checks positions; never read outside the tables
  const int half = rotary_dim >> 1;
  const uint16_t* cs = cos_table + tpos * half;
  const uint16_t* sn = sin_table + tpos * half;
  auto rotate = [&](const uint16_t* x, int d) -> uint16_t {
    if (d >= rotary_dim) return x[d];
    const int f = d < half ? d : d - half;
    const float c = elem_to_f32<XT>(cs[f]), sv = elem_to_f32<XT>(sn[f]), val = elem_to_f32<XT>(x[d]);
    const float r = d < half ? -elem_to_f32<XT>(x[d + half]) : elem_to_f32<XT>(x[d - half]);
    return f32_to_elem_bits<XT>(val * c + r * sv);
  };
  const int64_t q_elems = (int64_t)heads * dim, kv_elems = (int64_t)heads_kv * dim;
  const uint16_t* qs = q + t * q_elems;
  uint16_t* qd = q_rot + t * q_elems;
  const int64_t phys = addressable ? physical_token(block_table + (int64_t)b * bt_row_stride, pos, page_size, n_pages) : 0;
  const uint16_t* ks = k_new + t * kv_elems;
  const uint16_t* vs = v_new + t * kv_elems;
  uint16_t* kd = k_pages + phys * kv_elems;
  uint16_t* vd = v_pages + phys * kv_elems;
  if ((half & 1) == 0) {
    // two neighbouring pairs per work item, everything in 4-byte accesses: items [0, half/2) of a head rotate
    // (d, d+1, d+half, d+half+1), the rest copy the dimensions past rotary_dim two at a time
    const int rot_items = half >> 1;
    auto head_item = [&](const uint16_t* x, uint16_t* y, int it) {
      if (it >= rot_items) {
        const int d = rotary_dim + 2 * (it - rot_items);
        *(uint32_t*)(y + d) = *(const uint32_t*)(x + d);
        return;
      }
      const int d = 2 * it;
      uint32_t lo_raw[1] = {*(const uint32_t*)(x + d)}, hi_raw[1] = {*(const uint32_t*)(x + d + half)};
      uint32_t c_raw[1] = {*(const uint32_t*)(cs + d)}, s_raw[1] = {*(const uint32_t*)(sn + d)};
      float lo[2], hi[2], c[2], sv[2];
      Unpack<XT, 2>::run(lo_raw, lo);
      Unpack<XT, 2>::run(hi_raw, hi);
      Unpack<XT, 2>::run(c_raw, c);
      Unpack<XT, 2>::run(s_raw, sv);
      const uint32_t o_lo = (uint32_t)f32_to_elem_bits<XT>(lo[0] * c[0] + (-hi[0]) * sv[0]) |
                            ((uint32_t)f32_to_elem_bits<XT>(lo[1] * c[1] + (-hi[1]) * sv[1]) << 16);
      const uint32_t o_hi = (uint32_t)f32_to_elem_bits<XT>(hi[0] * c[0] + lo[0] * sv[0]) |
                            ((uint32_t)f32_to_elem_bits<XT>(hi[1] * c[1] + lo[1] * sv[1]) << 16);
      *(uint32_t*)(y + d) = o_lo;
      *(uint32_t*)(y + d + half) = o_hi;
    };
    const int items = rot_items + ((dim - rotary_dim) >> 1);  // per head: rotating items, then copying ones
    for (int i = threadIdx.x; i < heads * items; i += 256) {
      const int h = i / items, it = i - h * items;
      head_item(qs + (int64_t)h * dim, qd + (int64_t)h * dim, it);
    }
    if (!addressable) return;
    for (int i = threadIdx.x; i < heads_kv * items; i += 256) {
      const int h = i / items, it = i - h * items;
      head_item(ks + (int64_t)h * dim, kd + (int64_t)h * dim, it);
    }
    for (int64_t i = threadIdx.x * 2; i < kv_elems; i += 512) *(uint32_t*)(vd + i) = *(const uint32_t*)(vs + i);
    return;
  }
  for (int64_t i = threadIdx.x; i < q_elems; i += 256) {
    const int d = (int)(i % dim);
    qd[i] = rotate(qs + (i - d), d);
  }
  if (!addressable) return;
  for (int64_t i = threadIdx.x; i < kv_elems; i += 256) {
    const int d = (int)(i % dim);
    kd[i] = rotate(ks + (i - d), d);
    vd[i] = vs[i];
  }
}

const char* launch_rope_append_chunk(const void* q, const void* k_new, const void* v_new, void* q_rot, void* k_pages, void* v_pages,
                                     const void* cos_table, const void* sin_table, const int32_t* cu_q,
                                     const int32_t* cache_seqlens, const int32_t* block_table, int64_t bt_row_stride, int batch,
                                     int64_t total_q, int heads, int heads_kv, int dim, int rotary_dim, int64_t max_position,
                                     int page_size, int64_t n_pages, int x_dtype, hipStream_t s) {
  if (batch == 0 || total_q == 0) return nullptr;
#define MI355_LAUNCH_ROPE(XT)                                                                                                   \
  hipLaunchKernelGGL((rope_append_chunk_kernel<XT>), dim3((unsigned)total_q), dim3(256), 0, s, (const uint16_t*)q,              \
                     (const uint16_t*)k_new, (const uint16_t*)v_new, (uint16_t*)q_rot, (uint16_t*)k_pages, (uint16_t*)v_pages,   \
                     (const uint16_t*)cos_table, (const uint16_t*)sin_table, cu_q, cache_seqlens, block_table, bt_row_stride,   \
                     batch, heads, heads_kv, dim, rotary_dim, max_position, page_size, n_pages)
  if (x_dtype == MI355_DT_BF16) MI355_LAUNCH_ROPE(bf16_tag);
  else MI355_LAUNCH_ROPE(fp16_tag);
#undef MI355_LAUNCH_ROPE
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

// FP8 cache, prefill chunk: every sequence's keys (and values) as one contiguous run of 16-bit rows -- the cached tokens
// gathered through the block table and dequantised as the reference does, (fp8.float() * scale).to(dtype) with one scale
// per tensor (gqa_fwd.py:1063-1065), followed by the chunk's own tokens as they came.  Sequence b occupies rows
// [b*stride, b*stride + len_b) of kp / vp, len_b = the length the attention kernel will form from the same two arrays
// (seq_len_finish: cache length + chunk length, clamped to the slot); kv_starts[b] = b*stride is written here too.
// One pass of the 16-bit attention kernel over these rows then replaces a pass over the fp8 pages plus a pass over
// the chunk: the bytes are converted once per call instead of once per wave that reads them.
// grid (ceil(stride / 64), batch): a workgroup packs 64 token rows, eight elements (16 bytes of output) per thread.
template <typename XT>
__global__ __launch_bounds__(256) void dequant_pack_chunk_kernel(const uint8_t* __restrict__ k_pages, const uint8_t* __restrict__ v_pages,
                                                                 const uint16_t* __restrict__ k_new, const uint16_t* __restrict__ v_new,
                                                                 const float* __restrict__ k_scale, const float* __restrict__ v_scale,
                                                                 const int32_t* __restrict__ cu_q, const int32_t* __restrict__ cache_seqlens,
                                                                 const int32_t* __restrict__ block_table, int64_t bt_row_stride,
                                                                 uint16_t* __restrict__ kp, uint16_t* __restrict__ vp,
                                                                 int32_t* __restrict__ kv_starts, int64_t row_elems, int page_size,
                                                                 int64_t n_pages, int stride, int table_tokens, int tpt_shift) {
  const int b = blockIdx.y;
  if (blockIdx.x == 0 && threadIdx.x == 0) kv_starts[b] = b * stride;
  const int q0 = cu_q[b], ql = cu_q[b + 1] - q0;
  if (ql <= 0) return;  // no query rows: the attention kernel gives this sequence no tile
  int cached = cache_seqlens[b];
  cached = cached < 0 ? 0 : cached;
  const int len = cached > stride - ql ? stride : cached + ql;  // == seq_len_finish() with max_len = stride
  const int n_old = min(min(cached, len), table_tokens);        // (a corrupt length cannot run the gather past the table row)
  const int t_end = min(len, (int)(blockIdx.x + 1) * 64);
  const float sk = k_scale[0], sv = v_scale[0];
  const int32_t* bt_row = block_table + (int64_t)b * bt_row_stride;
  // tpt threads per token row (the power of two that covers row_elems / 8, at most 256), 256 / tpt rows per round.
  // Eight rounds at a time, every load of the eight issued before the first is used and none behind a per-row branch (in the one
  // block of a sequence that holds both kinds of row, a row reads a clamped neighbour of the other kind and drops it): the kernel moves a few bytes per thread per
  // round, so what it needs is loads in flight, not arithmetic.
  const int sub = threadIdx.x >> tpt_shift, lane_e = threadIdx.x & ((1 << tpt_shift) - 1), rows_per_round = 256 >> tpt_shift;
  const int per_row = (int)(row_elems / 8);
  constexpr int UN = 8;
  const int last_old = max(n_old - 1, 0);
  // pages of a multiple of 64 tokens: the workgroup's 64 tokens lie in one page, one table entry serves them all
  const bool one_page = (page_size & 63) == 0;
  const int blk0 = (int)blockIdx.x * 64;
  const int64_t phys_blk = physical_token(bt_row, min(blk0, last_old), page_size, n_pages) - min(blk0, last_old);
  // A block of 64 tokens is all cached tokens, all chunk tokens, or (one block per sequence) both: the loads a block has
  // no use for are not issued at all (the choice is the same for the whole workgroup).
  const bool any_old = blk0 < n_old, any_new = t_end > n_old;
  for (int c = lane_e; c < per_row; c += 1 << tpt_shift) {  // (one trip unless a row is wider than 256 threads x 8 elements)
    const int64_t e = (int64_t)c * 8;
    for (int t0 = blk0 + sub; t0 < t_end; t0 += UN * rows_per_round) {
      u32x2 kr[UN], vr[UN];
      uint4 kn[UN], vn[UN];
      if (any_old) {
        int64_t phys[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
          const int tc = min(t0 + u * rows_per_round, last_old);
          phys[u] = one_page ? phys_blk + tc : physical_token(bt_row, tc, page_size, n_pages);
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
          const int64_t src_old = phys[u] * row_elems + e;
          kr[u] = *(const u32x2*)(k_pages + src_old);
          vr[u] = *(const u32x2*)(v_pages + src_old);
        }
      }
      if (any_new) {
#pragma unroll
        for (int u = 0; u < UN; u++) {
          const int t = t0 + u * rows_per_round;
          const int64_t src_new = ((int64_t)q0 + min(max(t - cached, 0), ql - 1)) * row_elems + e;  // chunk token t - cached
          kn[u] = *(const uint4*)(k_new + src_new);
          vn[u] = *(const uint4*)(v_new + src_new);
        }
      }
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int t = t0 + u * rows_per_round;
        if (t >= t_end) continue;
        if (t < n_old) {
          const uint32_t kw[2] = {kr[u][0], kr[u][1]}, vw[2] = {vr[u][0], vr[u][1]};
          float kf[8], vf[8];
          Unpack<fp8_tag, 8>::run(kw, kf);
          Unpack<fp8_tag, 8>::run(vw, vf);
#pragma unroll
          for (int j = 0; j < 4; j++) {
            ((uint32_t*)&kn[u])[j] = (uint32_t)f32_to_elem_bits<XT>(kf[2 * j] * sk) | ((uint32_t)f32_to_elem_bits<XT>(kf[2 * j + 1] * sk) << 16);
            ((uint32_t*)&vn[u])[j] = (uint32_t)f32_to_elem_bits<XT>(vf[2 * j] * sv) | ((uint32_t)f32_to_elem_bits<XT>(vf[2 * j + 1] * sv) << 16);
          }
        }
        const int64_t dst = ((int64_t)b * stride + t) * row_elems + e;
        *(uint4*)(kp + dst) = kn[u];
        *(uint4*)(vp + dst) = vn[u];
      }
    }
  }
}

const char* launch_dequant_pack_chunk(const void* k_pages, const void* v_pages, const void* k_new, const void* v_new,
                                      const float* k_scale, const float* v_scale, const int32_t* cu_q, const int32_t* cache_seqlens,
                                      const int32_t* block_table, int64_t bt_row_stride, void* kp, void* vp, int32_t* kv_starts,
                                      int batch, int heads_kv, int dim, int page_size, int64_t n_pages, int stride, int x_dtype,
                                      hipStream_t s) {
  if (batch == 0) return nullptr;
  const int64_t row_elems = (int64_t)heads_kv * dim;  // a multiple of 64: head dims are
  const int64_t table_tokens64 = bt_row_stride * (int64_t)page_size;
  const int table_tokens = table_tokens64 > INT_MAX ? INT_MAX : (int)table_tokens64;
  int tpt_shift = 0;
  while ((1 << tpt_shift) < row_elems / 8 && tpt_shift < 8) ++tpt_shift;
  const dim3 grid((unsigned)((stride + 63) / 64), (unsigned)batch);
#define MI355_LAUNCH_PACK(XT)                                                                                                  \
  hipLaunchKernelGGL(dequant_pack_chunk_kernel<XT>, grid, dim3(256), 0, s, (const uint8_t*)k_pages, (const uint8_t*)v_pages,   \
                     (const uint16_t*)k_new, (const uint16_t*)v_new, k_scale, v_scale, cu_q, cache_seqlens, block_table,       \
                     bt_row_stride, (uint16_t*)kp, (uint16_t*)vp, kv_starts, row_elems, page_size, n_pages, stride, table_tokens, tpt_shift)
  if (x_dtype == MI355_DT_BF16) MI355_LAUNCH_PACK(bf16_tag);
  else MI355_LAUNCH_PACK(fp16_tag);
#undef MI355_LAUNCH_PACK
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

// Merge two attention results over disjoint key sets, given as fp32 rows with log2-domain log-sum-exp:
//   out = (2^(lse_a - m) * o_a + 2^(lse_b - m) * o_b) / (2^(lse_a - m) + 2^(lse_b - m)),  m = max(lse_a, lse_b);
// a row both sides left empty (-inf, -inf) becomes zero.  One thread per two head elements.
template <typename QT>
__global__ __launch_bounds__(256) void merge_two_kernel(const float* __restrict__ o_a, const float* __restrict__ lse_a,
                                                        const float* __restrict__ o_b, const float* __restrict__ lse_b,
                                                        uint32_t* __restrict__ out, int64_t rows, int half_dim) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * half_dim) return;
  const int64_t row = idx / half_dim;
  const float la = lse_a[row], lb = lse_b[row], m = fmaxf(la, lb);
  float r0 = 0.f, r1 = 0.f;
  if (m > -INFINITY) {
    const float wa = exp2f(la - m), wb = exp2f(lb - m), inv = 1.0f / (wa + wb);
    const f32x2 a = *(const f32x2*)(o_a + 2 * idx), b = *(const f32x2*)(o_b + 2 * idx);
    r0 = (wa != 0.f ? wa * a[0] : 0.f) + (wb != 0.f ? wb * b[0] : 0.f);
    r1 = (wa != 0.f ? wa * a[1] : 0.f) + (wb != 0.f ? wb * b[1] : 0.f);
    r0 *= inv;
    r1 *= inv;
  }
  out[idx] = (uint32_t)f32_to_elem_bits<QT>(r0) | ((uint32_t)f32_to_elem_bits<QT>(r1) << 16);
}

const char* launch_merge_two(const float* o_a, const float* lse_a, const float* o_b, const float* lse_b, void* out,
                             int64_t rows, int dim, int q_dtype, hipStream_t s) {
  if (rows == 0) return nullptr;
  const int64_t n = rows * (dim / 2);
  const unsigned grid = (unsigned)((n + 255) / 256);
  if (q_dtype == MI355_DT_BF16)
    hipLaunchKernelGGL(merge_two_kernel<bf16_tag>, dim3(grid), dim3(256), 0, s, o_a, lse_a, o_b, lse_b, (uint32_t*)out, rows, dim / 2);
  else
    hipLaunchKernelGGL(merge_two_kernel<fp16_tag>, dim3(grid), dim3(256), 0, s, o_a, lse_a, o_b, lse_b, (uint32_t*)out, rows, dim / 2);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

}  // namespace mi355
