// Generic paged GQA decode kernel for gfx950: fp32 VALU dot products, any page size, any GQA group,
// head_dim in {64, 128, 256}, bf16/fp16/fp8-e4m3fn KV, optional softcap and causal multi-token queries.
//
// It takes over what the reference's two TileLang kernels compute
// (src/tileops/kernels/attention/gqa_decode_paged.py:75-168 no-split, :209-342 split) plus the combine
// (:344-374), with these differences: split bounds come from each sequence's own length inside the kernel
// (no host read-back of max(real_seqlen_kv)), partial outputs and LSE are fp32, and the running maximum
// uses a finite floor so an empty split contributes weight 0 instead of NaN.
//
// Work decomposition: one workgroup of 256 threads = 16 groups of 16 lanes per (sequence, kv head,
// block of RB query rows, KV split).  A 16-lane group owns one token at a time: each lane holds D/16
// consecutive head elements (one 128-bit load for bf16 at D=128, so a wave instruction reads four whole
// 256-byte K rows), dots them against the RB query rows held in registers, and the 16 partial sums are
// reduced with four xor-shuffles.  Each group keeps its own online-softmax state; the 16 states are merged
// once at the end (shuffles inside a wave, LDS across the four waves).
#include "common.h"
#include "device_utils.h"

namespace mi355 {

template <int NBYTES> __device__ __forceinline__ void load_raw(const void* p, uint32_t* raw) {
  if constexpr (NBYTES == 4) {
    raw[0] = *(const uint32_t*)p;
  } else if constexpr (NBYTES == 8) {
    u32x2 v = *(const u32x2*)p;
    raw[0] = v[0];
    raw[1] = v[1];
  } else {
#pragma unroll
    for (int i = 0; i < NBYTES / 16; i++) {
      u32x4 v = ((const u32x4*)p)[i];
      raw[4 * i] = v[0];
      raw[4 * i + 1] = v[1];
      raw[4 * i + 2] = v[2];
      raw[4 * i + 3] = v[3];
    }
  }
}

template <typename QT, typename KVT, int D, int RB, bool SOFTCAP>
__global__ __launch_bounds__(256) void paged_decode_generic_kernel(const DecodeParams p) {
  constexpr int EPL = D / 16;  // head elements per lane
  constexpr int QB = ElemTraits<QT>::bytes, KB = ElemTraits<KVT>::bytes;
  constexpr bool FP8 = KB == 1;
  const int tid = threadIdx.x, c = tid & 15, gi = tid >> 4, wave = tid >> 6;
  const int n_rowblk = (p.rows + RB - 1) / RB;
  const int kvh = blockIdx.x / n_rowblk, r0 = (blockIdx.x % n_rowblk) * RB;
  const int split = blockIdx.y, b = blockIdx.z;
  const int len = seq_len_of(p, b);
  int n_splits, chunk;
  split_geometry(len, p.split_tokens, p.max_splits, &n_splits, &chunk);
  if (split >= n_splits) return;
  const int t_begin = split * chunk;
  const int t_end = min(len, t_begin + chunk);
  const int32_t* bt_row = p.block_table + (int64_t)b * p.bt_row_stride;

  const int q_len_b = q_len_of(p, b), rows_b = q_len_b * p.group;
  const int64_t q_row0 = q_row0_of(p, b);
  float qf[RB][EPL];
  int limit[RB];
#pragma unroll
  for (int rr = 0; rr < RB; rr++) {
    int r = r0 + rr;
    bool valid = r < rows_b;
    int s = valid ? r / p.group : 0, gidx = valid ? r % p.group : 0;
    const char* qp = (const char*)p.q + (((q_row0 + s) * p.heads + kvh * p.group + gidx) * D + c * EPL) * QB;
    uint32_t raw[EPL * QB / 4] = {};
    if (valid) load_raw<EPL * QB>(qp, raw);  // a row past the sequence's own rows may lie past the end of q
    Unpack<QT, EPL>::run(raw, qf[rr]);
    limit[rr] = valid ? ((p.causal && p.q_len > 1) ? len - q_len_b + s + 1 : len) : 0;
  }

  float m[RB], l[RB], acc[RB][EPL];
#pragma unroll
  for (int rr = 0; rr < RB; rr++) {
    m[rr] = kNegFloor;
    l[rr] = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; e++) acc[rr][e] = 0.f;
  }

  for (int t = t_begin + gi; t < t_end; t += 16) {
    const int64_t phys = p.kv_starts ? (int64_t)p.kv_starts[b] + t : p.contig_stride ? (int64_t)b * p.contig_stride + t : physical_token(bt_row, t, p.page_size, p.n_pages);
    const int64_t row = phys * p.heads_kv + kvh;
    uint32_t kraw[EPL * KB / 4], vraw[EPL * KB / 4];
    load_raw<EPL * KB>((const char*)p.k + (row * D + c * EPL) * KB, kraw);
    load_raw<EPL * KB>((const char*)p.v + (row * D + c * EPL) * KB, vraw);
    float ks = 1.f, vs = 1.f;
    if (FP8) {
      ks = p.k_scale[p.scale_per_tensor ? 0 : row];
      vs = p.v_scale[p.scale_per_tensor ? 0 : row];
    }
    float kf[EPL], vf[EPL];
    Unpack<KVT, EPL>::run(kraw, kf);
    Unpack<KVT, EPL>::run(vraw, vf);
#pragma unroll
    for (int rr = 0; rr < RB; rr++) {
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < EPL; e++) s = fmaf(qf[rr][e], kf[e], s);
      s += __shfl_xor(s, 1, 64);
      s += __shfl_xor(s, 2, 64);
      s += __shfl_xor(s, 4, 64);
      s += __shfl_xor(s, 8, 64);
      if (t < limit[rr]) {
        float x = to_logit2<SOFTCAP>(s * ks, p.score_scale, p.cap_log2e, p.inv_cap_scale);
        float m_new = fmaxf(m[rr], x);
        float alpha = exp2f(m[rr] - m_new);
        float pr = exp2f(x - m_new);
        l[rr] = l[rr] * alpha + pr;
        float pv = pr * vs;
#pragma unroll
        for (int e = 0; e < EPL; e++) acc[rr][e] = fmaf(acc[rr][e], alpha, pv * vf[e]);
        m[rr] = m_new;
      }
    }
  }

  // merge the four 16-lane groups of a wave
#pragma unroll
  for (int rr = 0; rr < RB; rr++) {
    float m_all = fmaxf(m[rr], __shfl_xor(m[rr], 16, 64));
    m_all = fmaxf(m_all, __shfl_xor(m_all, 32, 64));
    float sc = exp2f(m[rr] - m_all);
    float lv = l[rr] * sc;
    lv += __shfl_xor(lv, 16, 64);
    lv += __shfl_xor(lv, 32, 64);
    l[rr] = lv;
    m[rr] = m_all;
#pragma unroll
    for (int e = 0; e < EPL; e++) {
      float a = acc[rr][e] * sc;
      a += __shfl_xor(a, 16, 64);
      a += __shfl_xor(a, 32, 64);
      acc[rr][e] = a;
    }
  }
  // merge the four waves through LDS
  __shared__ float sm_m[4][RB], sm_l[4][RB];
  __shared__ float sm_acc[4][RB][D];
  if ((tid & 63) < 16) {
#pragma unroll
    for (int rr = 0; rr < RB; rr++) {
      if (c == 0) {
        sm_m[wave][rr] = m[rr];
        sm_l[wave][rr] = l[rr];
      }
#pragma unroll
      for (int e = 0; e < EPL; e++) sm_acc[wave][rr][c * EPL + e] = acc[rr][e];
    }
  }
  __syncthreads();
  const bool direct = n_splits == 1;
  for (int idx = tid; idx < RB * D; idx += 256) {
    int rr = idx / D, d = idx - rr * D;
    int r = r0 + rr;
    if (r >= rows_b) continue;
    float M = fmaxf(fmaxf(sm_m[0][rr], sm_m[1][rr]), fmaxf(sm_m[2][rr], sm_m[3][rr]));
    float L = 0.f, A = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) {
      float sc = exp2f(sm_m[w][rr] - M);
      L += sm_l[w][rr] * sc;
      A += sm_acc[w][rr][d] * sc;
    }
    float o = L > 0.f ? A / L : 0.f;
    int s = r / p.group, gidx = r % p.group;
    if (direct) {
      const int64_t orow = (q_row0 + s) * p.heads + kvh * p.group + gidx;
      if (p.final_o) {
        p.final_o[orow * D + d] = o;
        if (d == 0) p.final_lse[orow] = L > 0.f ? M + log2f(L) : -INFINITY;
      } else {
        *((uint16_t*)p.out + orow * D + d) = f32_to_elem_bits<QT>(o);
      }
    } else {
      // partial slot (b, split); rows of all kv heads side by side: global row = kvh*rows + r
      int64_t slot = (int64_t)b * p.max_splits + split;
      int64_t grow = slot * ((int64_t)p.heads_kv * p.rows) + (int64_t)kvh * p.rows + r;
      p.part_o[grow * D + d] = o;
      if (d == 0) p.part_lse[grow] = L > 0.f ? M + log2f(L) : -INFINITY;
    }
  }
}

// Combine of the generic kernel's partials: grid (heads_kv*rows, batch), D threads.
// lse = log2 sum_s 2^(lse_s - max) + max ; O = sum_s 2^(lse_s - lse) * O_s   (reference :344-374), fp32 in.
template <typename QT>
__global__ void paged_decode_generic_combine_kernel(const DecodeParams p) {
  const int b = blockIdx.y, grow_in = blockIdx.x, d = threadIdx.x;
  const int len = seq_len_of(p, b);
  int n_splits, chunk;
  split_geometry(len, p.split_tokens, p.max_splits, &n_splits, &chunk);
  if (n_splits == 1) return;  // the attention kernel wrote the output directly
  const int64_t rows_all = (int64_t)p.heads_kv * p.rows;
  float M = -INFINITY;
  for (int s = 0; s < n_splits; s++) M = fmaxf(M, p.part_lse[((int64_t)b * p.max_splits + s) * rows_all + grow_in]);
  float W = 0.f, A = 0.f;
  if (M > -INFINITY) {
    for (int s = 0; s < n_splits; s++) {
      int64_t grow = ((int64_t)b * p.max_splits + s) * rows_all + grow_in;
      float w = exp2f(p.part_lse[grow] - M);
      W += w;
      A += w * p.part_o[grow * p.dim + d];
    }
  }
  float o = W > 0.f ? A / W : 0.f;
  int kvh = grow_in / p.rows, r = grow_in % p.rows;
  if (r >= q_len_of(p, b) * p.group) return;  // packed queries: this sequence has fewer rows
  int s = r / p.group, gidx = r % p.group;
  const int64_t orow = (q_row0_of(p, b) + s) * p.heads + kvh * p.group + gidx;
  if (p.final_o) {
    p.final_o[orow * p.dim + d] = o;
    if (d == 0) p.final_lse[orow] = W > 0.f ? M + log2f(W) : -INFINITY;
  } else {
    *((uint16_t*)p.out + orow * p.dim + d) = f32_to_elem_bits<QT>(o);
  }
}

template <typename QT, typename KVT, int D, int RB>
static const char* launch_generic_t2(const DecodeParams& p, hipStream_t s) {
  int n_rowblk = (p.rows + RB - 1) / RB;
  dim3 grid(p.heads_kv * n_rowblk, p.max_splits, p.batch);
  if (p.softcap > 0.f)
    hipLaunchKernelGGL((paged_decode_generic_kernel<QT, KVT, D, RB, true>), grid, dim3(256), 0, s, p);
  else
    hipLaunchKernelGGL((paged_decode_generic_kernel<QT, KVT, D, RB, false>), grid, dim3(256), 0, s, p);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

template <typename QT, typename KVT>
static const char* launch_generic_t1(const DecodeParams& p, hipStream_t s) {
  const bool small = p.rows <= 4;
  switch (p.dim) {
    case 64:
      return small ? launch_generic_t2<QT, KVT, 64, 4>(p, s) : launch_generic_t2<QT, KVT, 64, 8>(p, s);
    case 128:
      return small ? launch_generic_t2<QT, KVT, 128, 4>(p, s) : launch_generic_t2<QT, KVT, 128, 8>(p, s);
    case 256:
      return small ? launch_generic_t2<QT, KVT, 256, 4>(p, s) : launch_generic_t2<QT, KVT, 256, 8>(p, s);
  }
  return "generic kernel: head dim must be 64, 128 or 256";
}

const char* launch_generic(const DecodeParams& p, int q_dtype, int kv_dtype, hipStream_t s) {
  if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_BF16) return launch_generic_t1<bf16_tag, bf16_tag>(p, s);
  if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP16) return launch_generic_t1<fp16_tag, fp16_tag>(p, s);
  if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_generic_t1<bf16_tag, fp8_tag>(p, s);
  if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_generic_t1<fp16_tag, fp8_tag>(p, s);
  return "generic kernel: unsupported (q_dtype, kv_dtype) pair";
}

const char* launch_generic_combine(const DecodeParams& p, int q_dtype, hipStream_t s) {
  if (p.max_splits <= 1) return nullptr;
  dim3 grid(p.heads_kv * p.rows, p.batch);
  if (q_dtype == MI355_DT_BF16)
    hipLaunchKernelGGL(paged_decode_generic_combine_kernel<bf16_tag>, grid, dim3(p.dim), 0, s, p);
  else
    hipLaunchKernelGGL(paged_decode_generic_combine_kernel<fp16_tag>, grid, dim3(p.dim), 0, s, p);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

}  // namespace mi355
