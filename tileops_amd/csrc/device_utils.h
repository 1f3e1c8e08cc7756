// Device-side helpers: element conversion, page arithmetic, wave-level reductions (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

struct bf16_tag {};
struct fp16_tag {};
struct fp8_tag {};

template <typename T> struct ElemTraits;
template <> struct ElemTraits<bf16_tag> { static constexpr int bytes = 2; };
template <> struct ElemTraits<fp16_tag> { static constexpr int bytes = 2; };
template <> struct ElemTraits<fp8_tag> { static constexpr int bytes = 1; };

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float fp16_bits_to_f32(uint32_t b) {
  _Float16 h;
  uint16_t u = (uint16_t)b;
  __builtin_memcpy(&h, &u, 2);
  return (float)h;
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  __bf16 h = (__bf16)f;  // round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
  uint16_t u;
  __builtin_memcpy(&u, &h, 2);
  return u;
}
__device__ __forceinline__ uint16_t f32_to_fp16_bits(float f) {
  _Float16 h = (_Float16)f;
  uint16_t u;
  __builtin_memcpy(&u, &h, 2);
  return u;
}

// Convert N consecutive elements (N*bytes <= 16, loaded as raw dwords) to fp32.
template <typename T, int N> struct Unpack;
template <int N> struct Unpack<bf16_tag, N> {
  __device__ static __forceinline__ void run(const uint32_t* raw, float* out) {
#pragma unroll
    for (int i = 0; i < N / 2; i++) {
      out[2 * i] = __uint_as_float(raw[i] << 16);
      out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
  }
};
template <int N> struct Unpack<fp16_tag, N> {
  __device__ static __forceinline__ void run(const uint32_t* raw, float* out) {
#pragma unroll
    for (int i = 0; i < N / 2; i++) {
      out[2 * i] = fp16_bits_to_f32(raw[i] & 0xffffu);
      out[2 * i + 1] = fp16_bits_to_f32(raw[i] >> 16);
    }
  }
};
template <int N> struct Unpack<fp8_tag, N> {
  __device__ static __forceinline__ void run(const uint32_t* raw, float* out) {
#pragma unroll
    for (int i = 0; i < N / 4; i++) {
      f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(raw[i], false);  // OCP e4m3fn on gfx950
      f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(raw[i], true);
      out[4 * i] = lo[0];
      out[4 * i + 1] = lo[1];
      out[4 * i + 2] = hi[0];
      out[4 * i + 3] = hi[1];
    }
  }
};

template <typename T> __device__ __forceinline__ uint16_t f32_to_elem_bits(float f);
template <> __device__ __forceinline__ uint16_t f32_to_elem_bits<bf16_tag>(float f) { return f32_to_bf16_bits(f); }
template <> __device__ __forceinline__ uint16_t f32_to_elem_bits<fp16_tag>(float f) { return f32_to_fp16_bits(f); }

// Logical token -> physical token through the block table.  The page id is clamped into the pool so
// that a corrupt table cannot make a kernel leave the allocation.
__device__ __forceinline__ int64_t physical_token(const int32_t* __restrict__ bt_row, int tok, int page_size,
                                                  int64_t n_pages) {
  int lp = tok / page_size;
  int64_t pg = bt_row[lp];
  pg = pg < 0 ? 0 : (pg >= n_pages ? n_pages - 1 : pg);
  return pg * page_size + (tok - lp * page_size);
}

// score (already multiplied by q.k) -> exp2-domain logit.
//   softcap off: x * (sm_scale*log2e) ; softcap on: cap*log2e * tanh(x * sm_scale/cap)
template <bool SOFTCAP>
__device__ __forceinline__ float to_logit2(float qk, float score_scale, float cap_log2e, float inv_cap_scale) {
  if (SOFTCAP) {
    // tanh(z) = 1 - 2/(exp(2z)+1) on the raw hardware exp2 and reciprocal (1 ulp each): exp2 saturates to 0 or +inf
    // and rcp(+inf) = 0, so both ends come out as exactly -1 and +1; the absolute error near zero is ~1e-7
    float e = __builtin_amdgcn_exp2f(qk * (inv_cap_scale * (2.0f * 1.4426950408889634f)));
    float t = __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(e + 1.0f), 1.0f);
    return cap_log2e * t;
  }
  return qk * score_scale;
}

__device__ __forceinline__ float wave_xor_max(float x, int mask) { return fmaxf(x, __shfl_xor(x, mask, 64)); }
__device__ __forceinline__ float wave_xor_sum(float x, int mask) { return x + __shfl_xor(x, mask, 64); }

}  // namespace mi355
