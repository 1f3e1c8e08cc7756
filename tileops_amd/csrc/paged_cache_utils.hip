// Page-table utilities for gfx950: the index-probe gather and the FP8 KV-cache append.
#include "common.h"
#include "device_utils.h"

namespace mi355 {

// One workgroup per (logical token, sequence): copy the physical row the block table names into the
// dense [batch, max_len, row_bytes] output.  Uses physical_token(), the page arithmetic shared with the
// attention kernels, so a bit-exact comparison against torch indexing pins that arithmetic.
__global__ void gather_probe_kernel(const uint32_t* __restrict__ cache, const int32_t* __restrict__ seqlens,
                                    const int32_t* __restrict__ block_table, int64_t bt_row_stride,
                                    uint32_t* __restrict__ dense_out, int64_t max_len, int64_t row_dwords,
                                    int page_size, int64_t n_pages) {
  const int b = blockIdx.y;
  const int len = seqlens[b];
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
  if (len <= 0) return;
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

}  // namespace mi355
