// MFMA paged GQA decode for gfx950 (MI355X): head dims 64, 128 and 256 with bf16/fp16 or FP8-e4m3fn KV.
//
// What it computes is the reference's split kernel + combine
// (src/tileops/kernels/attention/gqa_decode_paged.py:209-374): per (sequence, kv head), online softmax in
// the exp2 domain over the paged K/V rows, all query rows that share the kv head served from one read of
// K/V; partial results merged by log-sum-exp weights.  How it is organised is specific to CDNA4:
//
//  * Work unit = one wave.  A wave owns (partition, kv head, block of query rows) and runs on its own; only when a
//    kv head has several blocks of query rows do 2, 4 or 8 such waves share their LDS stages and meet at one
//    barrier per tile, or per two tiles on rings of four stages (see the kernel's template parameter SHW).  The KV "tile stream" (every 32-token tile of
//    every sequence, in batch order) is cut into n_parts equal contiguous ranges computed on the device from
//    real_seqlen_kv, so all
//    compute units get the same number of tiles whatever the length distribution, and nothing is read back
//    to the host.  A range that covers a whole sequence writes the output directly; a range that starts or
//    ends inside a sequence writes a partial row and its fp32 log-sum-exp (at most two per wave) that the combine kernel
//    merges; the rows are fp32, or the query's 16-bit type in multi-token calls with more than 4096 query rows (launch_mfma).
//  * Page gather = 128-bit direct-to-LDS loads (global_load_lds_dwordx4) with the non-temporal hint, 1 KiB
//    per wave instruction covering whole 128-, 256- or 512-byte K/V rows (head dim x element size), NS stages per wave in
//    flight, waited on with s_waitcnt vmcnt.  The LDS image is XOR-swizzled by choosing which 16-byte chunk
//    each lane fetches, so the reads below are bank-conflict free.
//  * QK^T: S^T[token][row] = K . Q^T on v_mfma_f32_16x16x32 (K rows straight from LDS as the A operand,
//    query rows resident in registers as B).  Having tokens on the M axis puts P in exactly the register
//    layout the PV product needs as its B operand, so P never moves between lanes.
//  * PV: O^T[d][row] += V^T . P^T, V^T fetched with LDS transpose reads (ds_read_b64_tr_b16 / _tr_b8).
//    Query rows sit on the N axis = lane % 16, so every per-row softmax quantity (max, sum, rescale factor)
//    is lane-local; the only cross-lane traffic is a two-step max/sum over the four 16-lane groups.
//  * FP8: V bytes are widened to bf16/fp16 on the LDS->register path (v_cvt_scalef32_pk_*_fp8, OCP e4m3fn).  At head
//    dims 128 and 256 the K bytes are not widened at all: Q.K^T runs on v_mfma_f32_16x16x128_f8f6f4 against the query
//    row split into two e4m3fn rows (hi + lo, exact for bf16 queries); at head dim 64 K is widened like V.
//    The per-token K scale multiplies the score and the V scale multiplies the probability, so no
//    head_dim-wide multiplies are spent on dequantisation.  Scales ride the same direct-to-LDS pipeline.
#include <atomic>

#include "common.h"
#include "device_utils.h"

namespace mi355 {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(8))) int i32x8;

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))
#define LDS_AT(T, addr) ((__attribute__((address_space(3))) T*)(uintptr_t)(addr))

constexpr int kCT = 32;       // tokens per pipeline stage (one MFMA K-block of the PV product)
constexpr int kD = 128;       // default head dim (64 and 256 also run)
// Single-row-block kernels with 128-byte rows (eight waves a CU) request the next tile only after the current one has
// landed; asking earlier keeps more requests in flight per CU than the memory system rewards (measured: -4 %).
constexpr bool kLateIssueNarrow = true;
// Shared rings of four stages consume two tiles per barrier where two tiles of one sequence are left: one wait and one
// barrier per 64 tokens instead of per 32.
constexpr bool kPairSteps = true;
constexpr bool kKPrefetch = true;

// Row groups (16*NRB query rows each) per kv head, and the same rounded up to whole rings of SHW waves: a ring may
// hold row groups past the last query row, which load nothing, mask everything and store nothing.
__host__ __device__ constexpr int row_groups(int rows, int nrb) { return (rows + 16 * nrb - 1) / (16 * nrb); }
__host__ __device__ constexpr int ring_row_groups(int rows, int nrb, int shw) { return (row_groups(rows, nrb) + shw - 1) / shw * shw; }
constexpr float kRescaleGap = 8.0f;  // see the lazy rescale in the softmax step

template <typename KVT, int D = kD> struct Geom {
  static constexpr bool FP8 = ElemTraits<KVT>::bytes == 1;
  static_assert(D == 64 || D == 128 || D == 256, "head dim 64, 128 or 256");
  static constexpr int ROW = D * ElemTraits<KVT>::bytes;   // bytes of one (token, kv head) row: 64, 128 or 256 (fp8), 128, 256 or 512 (16-bit)
  static constexpr int TPI = 1024 / ROW;                   // tokens per direct-to-LDS instruction
  static constexpr int NI = kCT / TPI;                     // instructions per K (or V) stage
  static constexpr int KBYTES = kCT * ROW;
  static constexpr int SCBYTES = FP8 ? 256 : 0;            // 32 K scales + 32 V scales
  static constexpr int STAGE = 2 * KBYTES + SCBYTES;
  static constexpr int IPS = 2 * NI + (FP8 ? 1 : 0);       // vector-memory instructions per stage
};

template <typename QT> struct Mma;
template <> struct Mma<bf16_tag> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {  // one v_cvt_pk_bf16_f32 (round to nearest even)
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
  }
  static __device__ __forceinline__ uint32_t from_fp8(uint32_t w, bool hi) {
    bf16x2 r = hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true) : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
    return __builtin_bit_cast(uint32_t, r);
  }
};
template <> struct Mma<fp16_tag> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {  // one v_cvt_pk_f16_f32 (round to nearest even)
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, f16x2));
  }
  static __device__ __forceinline__ uint32_t from_fp8(uint32_t w, bool hi) {
    f16x2 r = hi ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true) : __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
    return __builtin_bit_cast(uint32_t, r);
  }
};

template <typename QT> __device__ __forceinline__ f32x2 unpack2(uint32_t w);
template <> __device__ __forceinline__ f32x2 unpack2<bf16_tag>(uint32_t w) {
  return f32x2{__builtin_bit_cast(float, w << 16), __builtin_bit_cast(float, w & 0xffff0000u)};
}
template <> __device__ __forceinline__ f32x2 unpack2<fp16_tag>(uint32_t w) {
  return __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
}

// 16x16 tile of 128-deep dot products of e4m3fn bytes (v_mfma_f32_16x16x128_f8f6f4, no block scales): lane (c, g)
// supplies 32 bytes of row c of each operand.  Which 32 of the 128 depth positions those are is the same function of g
// for both operands, so any split of a row into four 32-byte parts may be used as long as both sides use the same.
__device__ __forceinline__ f32x4 mma_fp8_k128(u32x4 a_lo, u32x4 a_hi, u32x4 b_lo, u32x4 b_hi, f32x4 acc) {
  i32x8 a = {(int)a_lo[0], (int)a_lo[1], (int)a_lo[2], (int)a_lo[3], (int)a_hi[0], (int)a_hi[1], (int)a_hi[2], (int)a_hi[3]};
  i32x8 b = {(int)b_lo[0], (int)b_lo[1], (int)b_lo[2], (int)b_lo[3], (int)b_hi[0], (int)b_hi[1], (int)b_hi[2], (int)b_hi[3]};
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc, 0, 0, 0, 0, 0, 0);
}
// Four floats -> four e4m3fn bytes (round to nearest even; callers keep |x| <= 448).
__device__ __forceinline__ uint32_t pack_fp8x4(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
}

// 8 fp8 bytes (two dwords) -> 8 16-bit elements (four dwords), element order preserved.
template <typename QT> __device__ __forceinline__ u32x4 widen8(uint32_t w0, uint32_t w1) {
  u32x4 r;
  r[0] = Mma<QT>::from_fp8(w0, false);
  r[1] = Mma<QT>::from_fp8(w0, true);
  r[2] = Mma<QT>::from_fp8(w1, false);
  r[3] = Mma<QT>::from_fp8(w1, true);
  return r;
}

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const char* uni_ptr(const char* p) {
  uint64_t v = (uint64_t)p;
  uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const char*)(((uint64_t)hi << 32) | lo);
}

// Direct-to-LDS loads.  Issued through inline asm so that the waits are placed by hand (s_waitcnt vmcnt
// below): a stage may be consumed while later stages are still in flight.  M0 carries the LDS destination
// of lane 0; lane l lands at M0 + l*16 (or l*4).  The scalar operands are pinned to SGPRs here because a
// wave-uniform value may still have been computed on the vector ALU; the s_nop covers both the M0 write ->
// LDS-DMA wait state and the five wait states a VMEM instruction needs after a VALU write of its SGPR base,
// which the compiler's hazard recogniser cannot insert inside an asm block.
__device__ __forceinline__ void dma16_nt(uint32_t lds_addr, uint32_t voff, const char* sbase) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  sbase = uni_ptr(sbase);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void dma4(uint32_t lds_addr, const void* vaddr) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_addr), "v"(vaddr) : "memory");
}
template <int N> __device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// Reductions over the four 16-lane groups of a wave (lanes c, c+16, c+32, c+48) with the gfx950 lane-swap
// instructions: v_permlane16_swap exchanges odd 16-lane rows of its first operand with even rows of the
// second, v_permlane32_swap exchanges the upper half of the first with the lower half of the second.  Fed the
// same value twice they return (x of the even partner, x of the odd partner), so one max/add finishes a step
// without touching the LDS crossbar.
// Maxima as single instructions.  fmaxf() first quiets a possible signalling NaN in each operand whose origin
// the compiler cannot see (one extra v_max per operand); the scores here are MFMA results or -inf.
__device__ __forceinline__ float max2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float group_max(float x) {
  u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = max2(__uint_as_float(r[0]), __uint_as_float(r[1]));
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return max2(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float group_sum(float x) {
  u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// v_exp_f32: exp2 without the denormal-range fix-up of exp2f (arguments here are <= 0 or -inf; a result
// below 2^-126 may flush to zero, which is what a softmax weight that small should be).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Inclusive prefix sum over the 64 lanes on the data-parallel-primitive path (no LDS crossbar): four shifts inside each row
// of 16 lanes, then lane 15 of rows 0 and 2 added to rows 1 and 3, then lane 31 to rows 2 and 3.
__device__ __forceinline__ int wave_incl_scan(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);  // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);  // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);  // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);  // row_shr:8
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return x;
}

__device__ __forceinline__ int units_of(int len) { return (len + kCT - 1) / kCT; }

// Partition bounds u0(p) = floor(p*T/NP) (the merge kernels; the attention kernel forms the same numbers in 32 bits).
__device__ __forceinline__ int part_begin(int64_t p, int64_t T, int64_t NP) { return (int)(p * T / NP); }

// Position in the tile stream: sequence b, tile j of nt, plus the logical page / in-page offset of tile j.
// lens holds seqlens[lens_base + lane]: moving to the next sequence is a register read (v_readlane), not a global
// load whose wait would also drain every direct-to-LDS load in flight.
struct Cursor {
  int b, j, nt, len, pg, off;
  int lens_base, lens;
};

__device__ __forceinline__ void cursor_load_lens(Cursor& c, const DecodeParams& p, int base) {
  const int lane = threadIdx.x & 63;
  c.lens_base = base;
  c.lens = seq_len_of<true>(p, min(base + lane, p.batch - 1));
  // Land the load here.  Left to itself the compiler waits for it where the register is next read -- after the
  // join with the path that did not load, i.e. on every pass -- and its wait (vmcnt 0) also drains every
  // direct-to-LDS load in flight.  An empty asm that reads the register moves the wait into this rare block.
  asm volatile("" : "+v"(c.lens));
}

__device__ __forceinline__ void cursor_next(Cursor& c, const DecodeParams& p, bool ps16) {
  const int batch = p.batch, page_size = p.page_size;
  c.j++;
  if (c.j < c.nt) {
    if (ps16) {
      c.pg += 2;
    } else {
      c.off += kCT;
      if (c.off >= page_size) {
        c.off = 0;
        c.pg++;
      }
    }
    return;
  }
  c.j = 0;
  c.pg = 0;
  c.off = 0;
  do {
    c.b++;
    if (c.b >= batch) {
      c.nt = 0;
      c.len = 0;
      return;
    }
    if (c.b - c.lens_base >= 64) cursor_load_lens(c, p, c.b);  // once per 64 sequences
    c.len = __builtin_amdgcn_readlane(c.lens, c.b - c.lens_base);
    c.nt = units_of(c.len);
  } while (c.nt == 0);
}

// ------------------------------------------------------------------------------------------------------
// SHW > 1 (shared stages): when the row groups of a kv head come in multiples of SHW, a workgroup is SHW waves that
// serve SHW consecutive row groups of the same (partition, kv head), i.e. they walk the same tiles.  They share one
// LDS ring: each fetches 1/SHW of every stage, and one barrier per step (one tile, or two on a ring of four stages at
// head dims up to 128) makes all parts visible and retires the slots that are refilled next.  All waves execute the same
// number of barriers because they own the same tile range.
template <typename QT, typename KVT, int NRB, int NS, int NW, int SHW, int D>
__global__ __launch_bounds__(NW * 64, (SHW > 1 && (D <= 128 || SHW == 8)) ? 2 : 1) void paged_decode_mfma_kernel(const DecodeParams p, int* __restrict__ ws_prefix) {
  using G = Geom<KVT, D>;
  constexpr bool FP8 = G::FP8;
  constexpr int NJ = D / 32;    // 32-wide steps of the head dim in Q.K^T
  constexpr int NDB = D / 16;   // 16-wide blocks of the head dim in the output
  constexpr bool ROW128 = G::ROW == 128;        // 128-byte rows: fp8, or 16-bit with head dim 64 (8 KiB stages, eight waves a CU)
  constexpr bool R128 = ROW128 && !FP8;         // 16-bit rows of 128 bytes: the fp8 K layout with 16-bit elements
  constexpr bool ROW64 = G::ROW == 64;          // fp8 with head dim 64: 4.25 KiB stages, two fetch instructions per K tile
  constexpr bool F256 = FP8 && G::ROW == 256;   // fp8 with head dim 256: the 16-bit K layout of 256-byte rows, its own V^T layout
  // Q.K^T on the fp8 matrix instruction (one 128-deep step per 128 head elements): the K bytes go in as they are, the query
  // row goes in as two e4m3fn rows hi + lo (hi = the row times a power of two, rounded; lo = what the rounding dropped,
  // rounded again: exact for bf16 queries, within 2^-8 of every fp16 element) and the power of two multiplies the
  // softmax exponent.
  constexpr bool QK8 = FP8 && D >= 128;
  constexpr int NCH = D / 64;  // QK8: 16-byte chunks of a row per lane (chunk j = head elements [64j + 16g, 64j + 16g + 16))
  constexpr bool SH = SHW > 1;
  static_assert(!SH || (NW == SHW && G::NI % SHW == 0), "a shared-stage workgroup is the SHW waves of one ring");
  // Where the next fetch goes out: ahead of the wait for the current tile (one more stage in flight while waiting),
  // or after it (a tile lands before the next is requested: fewer requests in flight per compute unit).
  constexpr bool LATE = SH || (Geom<KVT, D>::ROW <= 128 && NRB == 1 && kLateIssueNarrow);
  constexpr int NIW = G::NI / SHW;                     // K (or V) fetch instructions per stage issued by this wave
  constexpr int IPSW = 2 * NIW + (FP8 ? 1 : 0);        // vector-memory instructions per stage issued by this wave
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int lane = threadIdx.x & 63;
  const int c = lane & 15, g = lane >> 4;
  const int wave = uni(threadIdx.x >> 6);
  // Workgroups are dealt round-robin to the 8 XCDs, so neighbouring partitions (which read neighbouring pages of
  // a sequence) spread over all L2s and memory channels; renumbering them XCD-contiguously measured slower.
  const int gw = blockIdx.x * NW + wave;
  const int n_rg = ring_row_groups(p.rows, NRB, SHW);
  const int per_part = p.heads_kv * n_rg;
  // integer division runs on the vector ALU; pin the results to scalar registers so that everything derived
  // from them (pool base pointers, LDS bases) is scalar arithmetic
  int part_, kvh_, rg_;
  if constexpr (SH) {
    // Workgroup g runs on XCD g % 8.  The workgroups of one (partition, kv head) read the same tiles and go to one XCD,
    // i.e. one L2.  Such groups are numbered kv-head-major, so with many partitions the kv heads of a partition (same
    // pages, shared 32-byte sectors of the scale rows) also meet on one XCD and neighbouring partitions land on
    // different ones, while a call with few partitions still spreads over all eight.
    const int per_group = n_rg / SHW, x = blockIdx.x & 7, y = blockIdx.x >> 3;  // workgroups per (partition, kv head)
    const int gid = x + 8 * (y / per_group);
    kvh_ = gid / p.n_parts;
    part_ = kvh_ < p.heads_kv ? gid - kvh_ * p.n_parts : p.n_parts;  // groups past the last: leave below
    rg_ = SHW * (y % per_group) + wave;
  } else {
    part_ = gw / per_part;
    kvh_ = (gw - part_ * per_part) / n_rg;
    rg_ = gw - part_ * per_part - kvh_ * n_rg;
  }
  const int part = uni(part_);
  const int kvh = uni(kvh_);
  const int rg = uni(rg_);
  const bool ps16 = p.page_size == 16;

  // ---- tile-stream bookkeeping: total tiles, this partition's range, first sequence of the range ------
  // One pass over the lengths (the first 64 stay in registers: with up to 64 sequences nothing is loaded twice), prefix
  // sums inside the wave on the data-parallel-primitive path, partition bounds in 32-bit arithmetic.  Everything a wave
  // does before its first K/V fetch is latency that no other wave of the compute unit hides: all of them are here too.
  int T = 0;
  int lens0 = 0, n0 = 0, incl0 = 0;
  for (int base = 0; base < p.batch; base += 64) {
    const int b = base + lane;
    const int len = b < p.batch ? seq_len_of<true>(p, b) : 0;
    const int n = units_of(len);
    const int incl = wave_incl_scan(n);
    if (base == 0) {
      lens0 = len;
      n0 = n;
      incl0 = incl;
    }
    T += __builtin_amdgcn_readlane(incl, 63);
  }
  T = uni(T);
  // bounds u0(p) = floor(p*T/NP) = p*(T/NP) + floor(p*(T%NP)/NP): the second product stays below NP^2 <= 2^24
  const uint32_t NPu = (uint32_t)p.n_parts, Tq = (uint32_t)T / NPu, Tr = (uint32_t)T - Tq * NPu;
  auto bound = [&](uint32_t pp) __attribute__((always_inline)) -> int { return (int)(pp * Tq + (pp * Tr) / NPu); };
  if (gw == 0) {
    // Per-sequence record for the combine kernel: {first tile, first partition, last partition, whether the
    // first partition holds this sequence in its second partial slot}.  Entry [batch] = {T, 0, 0, 0}.
    // Partition of tile u = the largest p with bound(p) <= u: a float estimate, off by at most one, put right by bound().
    const float np_over_t = (float)NPu / (float)(T > 0 ? T : 1);
    auto owner = [&](int u) __attribute__((always_inline)) -> int {
      int pp = min(max((int)((float)(u + 1) * np_over_t) - 1, 0), (int)NPu - 1);
#pragma unroll
      for (int i = 0; i < 2; i++)
        if (bound((uint32_t)pp) > u) --pp;
#pragma unroll
      for (int i = 0; i < 3; i++)
        if (pp + 1 < (int)NPu && bound((uint32_t)pp + 1) <= u) ++pp;
      return pp;
    };
    int carry = 0;
    for (int base = 0; base < p.batch; base += 64) {
      const int b = base + lane;
      int n = n0, incl = incl0;
      if (base > 0) {
        n = b < p.batch ? units_of(seq_len_of<true>(p, b)) : 0;
        incl = wave_incl_scan(n);
      }
      if (b < p.batch) {
        int pre = carry + incl - n;
        int4 rec = {pre, -1, -1, 0};  // y < 0 marks an empty sequence
        if (n > 0) {
          rec.y = owner(pre);
          rec.z = owner(pre + n - 1);
          rec.w = (bound((uint32_t)rec.y) != pre ? 1 : 0) | (T < (int)NPu ? 2 : 0);  // bit 1: some partitions own no tile
        }
        ((int4*)ws_prefix)[b] = rec;
      }
      carry += __builtin_amdgcn_readlane(incl, 63);
    }
    if (lane == 0) ((int4*)ws_prefix)[p.batch] = int4{T, 0, 0, 0};
  }
  if (part >= p.n_parts || T == 0) return;
  const int u0 = bound((uint32_t)part), u1 = bound((uint32_t)part + 1);
  const int n_units = u1 - u0;
  if (n_units <= 0) return;

  Cursor start;
  {
    int carry = 0, b0 = -1, pre0 = 0;
    start.lens = lens0;
    start.lens_base = 0;
    for (int base = 0; base < p.batch && b0 < 0; base += 64) {
      const int b = base + lane;
      int len = lens0, n = n0, incl = incl0;
      if (base > 0) {
        len = b < p.batch ? seq_len_of<true>(p, b) : 0;
        n = units_of(len);
        incl = wave_incl_scan(n);
      }
      const uint64_t hit = __ballot(carry + incl > u0);
      if (hit) {
        const int idx = uni(__ffsll((unsigned long long)hit) - 1);
        b0 = base + idx;
        pre0 = carry + __builtin_amdgcn_readlane(incl - n, idx);
        start.lens = len;  // lane l = sequence base + l: the cursor starts on registers already here
        start.lens_base = base;
      }
      carry += __builtin_amdgcn_readlane(incl, 63);
    }
    b0 = uni(b0);
    pre0 = uni(pre0);
    start.b = b0;
    start.len = __builtin_amdgcn_readlane(start.lens, b0 - start.lens_base);
    start.nt = units_of(start.len);
    start.j = u0 - pre0;
    if (ps16) {
      start.pg = 2 * start.j;
      start.off = 0;
    } else {
      int tok = start.j * kCT;
      start.pg = uni(tok / p.page_size);
      start.off = tok - start.pg * p.page_size;
    }
  }

  // ---- loop-invariant lane constants ------------------------------------------------------------------
  const uint32_t row_stride = (uint32_t)p.heads_kv * G::ROW;  // bytes between consecutive tokens of the pool
  const uint32_t lds_wave = uni((uint32_t)(size_t)LDS_PTR(char, smem)) + (SH ? 0 : wave) * (NS * G::STAGE);
  const int i0 = SH ? wave * NIW : 0;  // first of the NIW K (and V) fetch instructions of a stage that this wave issues

  // Direct-to-LDS source offsets.  Lane l of instruction i lands at LDS i*1024 + l*16, i.e. token
  // t = i*TPI + l/LPT (LPT lanes per token row), 16-byte slot l%LPT of that row.  The chunk fetched into
  // slot s of token t is s ^ f(t), with f chosen per operand so that the MFMA-layout reads are conflict free:
  //   16-bit, 256/512-byte rows  K: f = t%16   V: f = 2*(t%8)      (a 512-byte row: within each 256-byte half)
  //   16-bit, 128-byte rows  K: f = (t/2)%8    V: f = 2*((t/2)%4)
  //   fp8 (128-byte rows)    K: f = (t/2)%8    V: f = (t/2)%4 + 4*((t/16)%2)
  //   fp8 (64-byte rows)     K: f = (t/4)%4    V: f = (t/4)%2 + 2*((t/16)%2)
  //   fp8 (256-byte rows)    K: f = t%16       V: f = t%8 + 8*((t/16)%2)
  constexpr int LPT = G::ROW / 16;  // lanes per token row: 32, 16, 8 or 4
  // With 256-byte (512-byte) rows the patterns repeat every 4 (8) instructions for K and 2 (4) for V; with 128-byte
  // rows every 2 (K), and V is the same for all (16-bit) or changes once half way (fp8); with 64-byte rows K is the
  // same for both instructions and V differs between them.  A wave keeps one offset register per distinct pattern
  // among the instructions it issues.
  const int ts = lane / LPT, slot = lane % LPT;
  constexpr int PK = ROW64 ? 1 : (ROW128 ? 2 : 16 / G::TPI), PV = 8 / G::TPI;  // pattern periods (PV: wide 16-bit rows only)
  constexpr int NKO = NIW < PK ? NIW : PK;
  constexpr int NVO = F256 ? (NIW == 8 ? 4 : 2) : ROW64 ? NIW : (FP8 ? (NIW == 4 ? 2 : 1) : (R128 ? 1 : (NIW < PV ? NIW : PV)));
  uint32_t voff_k[NKO], voff_v[NVO];
#pragma unroll
  for (int e = 0; e < NKO; e++) {
    const int i = i0 + e;
    voff_k[e] = ts * row_stride + (ROW64 ? ((slot ^ ((ts / 4) & 3)) << 4)
                                         : (ROW128 ? ((slot ^ ((4 * i + ts / 2) & 7)) << 4) : ((slot ^ ((G::TPI * i + ts) & 15)) << 4)));
  }
#pragma unroll
  for (int e = 0; e < NVO; e++) {
    const int i = F256 ? (NIW == 8 ? (e & 1) + 4 * (e >> 1) : i0 + e) : (FP8 && !ROW64) ? (NIW == 4 ? 2 * e : i0) : i0 + e;
    voff_v[e] = ts * row_stride + (F256 ? ((slot ^ (((4 * i + ts) & 7) + 8 * ((i >> 2) & 1))) << 4)
                                   : ROW64 ? ((slot ^ (((ts / 4) & 1) + 2 * (i & 1))) << 4)
                                   : FP8 ? ((slot ^ (((ts / 2) & 3) + 4 * ((i >> 1) & 1))) << 4)
                                         : (R128 ? ((slot ^ (2 * ((ts / 2) & 3))) << 4) : ((slot ^ (2 * ((G::TPI * i + ts) & 7))) << 4)));
  }
  auto k_sel = [](int ii) __attribute__((always_inline)) { return ii % NKO; };
  auto v_sel = [](int ii) __attribute__((always_inline)) {
    if (F256) return NIW == 8 ? (ii & 1) + 2 * ((ii >> 2) & 1) : ii % NVO;
    return (FP8 && !ROW64) ? (NIW == 4 ? (ii >> 1) & 1 : 0) : ii % NVO;
  };

  // Absolute LDS read addresses of stage slot 0; slot s and token block tb are added as immediates.
  constexpr int NKA = ROW64 ? 1 : (ROW128 ? 2 : 4);
  uint32_t kaddr[NKA], vaddr[F256 ? 16 : (NDB < 8 ? NDB : 8)];  // (512-byte rows: the second 256 bytes are reached with an immediate)
  if constexpr (R128) {
    // head dim 64: K rows of 128 bytes read exactly like the fp8 K rows (16-byte chunk g + 4j of row c), V^T like the
    // 256-byte-row case with four 32-byte slots per row instead of eight
#pragma unroll
    for (int j = 0; j < 2; j++) kaddr[j] = lds_wave + (uint32_t)(c * 128 + (((g + 4 * j) ^ (c >> 1)) & 7) * 16);
    const int tk = 4 * g + c / 4;
#pragma unroll
    for (int db = 0; db < NDB; db++) vaddr[db] = lds_wave + G::KBYTES + (uint32_t)((tk * 128 + ((tk >> 1) & 3) * 32 + (c & 3) * 8) ^ (db * 32));
  } else if constexpr (!FP8) {
#pragma unroll
    for (int j = 0; j < 4; j++) kaddr[j] = lds_wave + (uint32_t)(c * G::ROW + (((4 * j + g) ^ c) & 15) * 16);
    const int tk = 4 * g + c / 4;  // transpose read: lane supplies row tk, 8 bytes at column group c%4
#pragma unroll
    for (int db = 0; db < 8; db++) vaddr[db] = lds_wave + G::KBYTES + (uint32_t)((tk * G::ROW + (tk & 7) * 32 + (c & 3) * 8) ^ (db * 32));
  } else if constexpr (F256) {
    // fp8, head dim 256: K chunks 4j + g of token row c as for 16-bit rows of this width; V^T bytes of sixteen rows per
    // half wave, one 16-byte chunk each, spread over all banks by f = t%8 + 8*((t/16)%2)
#pragma unroll
    for (int j = 0; j < 4; j++) kaddr[j] = lds_wave + (uint32_t)(c * 256 + (((4 * j + g) ^ c) & 15) * 16);
    const int r8 = c >> 1;
    const int tk = r8 < 4 ? 4 * g + r8 : 16 + 4 * g + (r8 - 4);
    const int fv = (tk & 7) + 8 * ((tk >> 4) & 1);
#pragma unroll
    for (int db = 0; db < 16; db++) vaddr[db] = lds_wave + G::KBYTES + (uint32_t)((tk * 256 + fv * 16 + (c & 1) * 8) ^ (db * 16));
  } else if constexpr (ROW64) {
    // fp8, head dim 64: lane (c, g) reads the 16 bytes of chunk g of token row c, i.e. both 8-wide k-steps of its group
    kaddr[0] = lds_wave + (uint32_t)(c * 64 + ((g ^ (c >> 2)) & 3) * 16);
    const int r8 = c >> 1;
    const int tk = r8 < 4 ? 4 * g + r8 : 16 + 4 * g + (r8 - 4);
    const int fv = ((tk >> 2) & 1) + 2 * ((tk >> 4) & 1);
#pragma unroll
    for (int db = 0; db < NDB; db++) vaddr[db] = lds_wave + G::KBYTES + (uint32_t)((tk * 64 + fv * 16 + (c & 1) * 8) ^ (db * 16));
  } else {
#pragma unroll
    for (int j = 0; j < 2; j++) kaddr[j] = lds_wave + (uint32_t)(c * 128 + (((g + 4 * j) ^ (c >> 1)) & 7) * 16);
    const int r8 = c >> 1;  // transpose read of bytes: lane supplies row r8 of 8, 8 bytes at half c%2
    const int tk = r8 < 4 ? 4 * g + r8 : 16 + 4 * g + (r8 - 4);
    const int fv = ((tk >> 1) & 3) + 4 * ((tk >> 4) & 1);
#pragma unroll
    for (int db = 0; db < 8; db++) vaddr[db] = lds_wave + G::KBYTES + (uint32_t)((tk * 128 + fv * 16 + (c & 1) * 8) ^ (db * 16));
  }
  const uint32_t saddr = lds_wave + 2 * G::KBYTES + (uint32_t)(4 * g) * 4;  // scales of tokens 4g.. (fp8)

  // ---- stage issue --------------------------------------------------------------------------------------
  const char* const kpool = uni_ptr((const char*)p.k + (int64_t)kvh * G::ROW);
  const char* const vpool = uni_ptr((const char*)p.v + (int64_t)kvh * G::ROW);
  // Block-table entries of the sequence being issued live in one VGPR: lane l holds logical page
  // bt_base + l.  A stage fetches its entry with v_readlane, so the steady-state loop contains no
  // compiler-visible memory load (whose vmcnt wait would drain the direct-to-LDS pipeline); the register
  // is refilled once per 64 pages.
  int bt_reg = 0, bt_base = 0, bt_seq = -1;
  int kvs_seq = -1;
  uint32_t kvs_val = 0;  // kv_starts[kvs_seq], fetched once per sequence
  const int last_page_id = (int)p.n_pages - 1;
  auto phys_page = [&](const Cursor& cu, int pg) __attribute__((always_inline)) -> int {
    if (cu.b != bt_seq || pg < bt_base || pg >= bt_base + 64) {
      bt_seq = cu.b;
      bt_base = pg;
      int last_pg = uni((cu.len - 1) / p.page_size);  // never read past the entries the sequence owns
      bt_reg = p.block_table[(int64_t)cu.b * p.bt_row_stride + min(pg + lane, last_pg)];
      asm volatile("" : "+v"(bt_reg));  // wait for it here, not after the join (see cursor_load_lens)
    }
    int e = __builtin_amdgcn_readlane(bt_reg, pg - bt_base);
    return min(max(e, 0), last_page_id);
  };
  // Row of the pool (physical token) that holds the first token of cu's tile.  The pool has fewer than 2^31 rows
  // (checked by the launcher).  Tiles inside one page, or one contiguous sequence, follow each other 32 rows apart,
  // so the issue cursor only comes here at page and sequence borders.  Not used with 16-token pages.
  const bool paged = !p.kv_starts && !p.contig_stride;
  auto locate = [&](const Cursor& cu) __attribute__((always_inline)) -> uint32_t {
    const int tok0 = cu.j * kCT;
    if (p.kv_starts) {  // packed contiguous keys: sequence b starts at kv_starts[b]
      if (cu.b != kvs_seq) {
        kvs_seq = cu.b;
        kvs_val = (uint32_t)uni(p.kv_starts[cu.b]);
      }
      return kvs_val + tok0;
    }
    if (p.contig_stride) return (uint32_t)cu.b * (uint32_t)p.contig_stride + tok0;  // contiguous cache: no table
    return (uint32_t)phys_page(cu, cu.pg) * (uint32_t)p.page_size + cu.off;
  };
  // fp8 scales of a full tile: lane l fetches the K (l < 32) or V scale of token l % 32; everything but the tile's
  // row is folded into a per-lane pointer once
  const uint32_t scale_row_bytes = p.scale_per_tensor ? 0u : (uint32_t)p.heads_kv * 4u;
  const char* const scale_lane = (const char*)(lane < 32 ? p.k_scale : p.v_scale) +
                                 (p.scale_per_tensor ? 0 : ((int64_t)(lane & 31) * p.heads_kv + kvh) * 4);
  auto issue = [&](const Cursor& cu, int slot_idx, uint32_t prow) __attribute__((always_inline)) {
    const int tok0 = cu.j * kCT;
    const int nvalid = min(kCT, cu.len - tok0);  // >= 1
    const uint32_t lds_stage = lds_wave + slot_idx * G::STAGE;
    const uint32_t lds = lds_stage + i0 * 1024;
    if (nvalid == kCT && !ps16) {
      // common case: 32 valid tokens inside one page -- straight-line, two scalar adds per instruction
      const uint64_t boff = (uint64_t)(prow + i0 * G::TPI) * row_stride;
      const char* kb = kpool + boff;
      const char* vb = vpool + boff;
      const uint32_t step = G::TPI * row_stride;
#pragma unroll
      for (int i = 0; i < NIW; i++) {
        dma16_nt(lds + i * 1024, voff_k[k_sel(i)], kb + i * step);
        dma16_nt(lds + G::KBYTES + i * 1024, voff_v[v_sel(i)], vb + i * step);
      }
      if (FP8) dma4(lds_stage + 2 * G::KBYTES, scale_lane + (uint64_t)prow * scale_row_bytes);  // (every wave of a ring: same bytes, same place)
      return;
    }
    // tail of a sequence and/or 16-token pages: rows past the valid ones re-read the last valid row, so
    // nothing outside (block_table, real_seqlen_kv) is ever touched
    int64_t ptok0 = prow, ptok1 = 0;  // physical token of the stage's first token (and of its second 16-token page)
    if (ps16) {
      int last_pg = (cu.len - 1) >> 4;
      ptok0 = (int64_t)phys_page(cu, cu.pg) * 16;
      ptok1 = (int64_t)phys_page(cu, min(cu.pg + 1, last_pg)) * 16;
    }
    const int i_last = (nvalid - 1) / G::TPI, t_last = (nvalid - 1) % G::TPI;
    constexpr int IPP = 16 / G::TPI;  // instructions per 16-token page
#pragma unroll
    for (int i = 0; i < NIW; i++) {
      int si = min(i + i0, i_last);
      int64_t ptok = ps16 ? (si < IPP ? ptok0 : ptok1) + (si % IPP) * G::TPI : ptok0 + si * G::TPI;
      uint32_t vk = voff_k[k_sel(i)], vv = voff_v[v_sel(i)];
      if (si == i_last && ts > t_last) {  // (also every instruction past i_last: si is clamped)
        uint32_t back = (uint32_t)(ts - t_last) * row_stride;
        vk -= back;
        vv -= back;
      }
      dma16_nt(lds + i * 1024, vk, kpool + ptok * row_stride);
      dma16_nt(lds + G::KBYTES + i * 1024, vv, vpool + ptok * row_stride);
    }
    if (FP8) {
      int tk = min(lane & 31, nvalid - 1);
      int64_t ptok = ps16 ? (tk < 16 ? ptok0 + tk : ptok1 + tk - 16) : ptok0 + tk;
      const float* sp = (lane < 32 ? p.k_scale : p.v_scale) + (p.scale_per_tensor ? 0 : ptok * p.heads_kv + kvh);
      dma4(lds_stage + 2 * G::KBYTES, sp);
    }
  };

  // ---- per-segment state ----------------------------------------------------------------------------------
  u32x4 qreg[NRB][NJ];
  f32x4 o_acc[NRB][NDB];
  float m_run[NRB], l_run[NRB];
  int limit[NRB];
  const int qoff = (p.causal && p.q_len > 1) ? p.q_len - 1 : 0;
  const bool softcap = p.softcap > 0.f;
  const uint32_t q_sign = p.negate_q ? (QK8 ? 0x80808080u : 0x80008000u) : 0u;
  float q_scale[NRB];  // QK8: the power of two taken out of the lane's query row (row c of each row block)

  int seg_q_len = p.q_len;   // query tokens of the sequence being processed (varies with packed queries)
  int64_t seg_q_row0 = 0;    // its first row in q / out
  auto begin_segment = [&](const Cursor& cu) __attribute__((always_inline)) {
    seg_q_len = uni(q_len_of(p, cu.b));
    seg_q_row0 = (int64_t)uni((int)q_row0_of(p, cu.b));
#pragma unroll
    for (int rb = 0; rb < NRB; rb++) {
      int r = rg * (16 * NRB) + rb * 16 + c;
      bool valid = r < seg_q_len * p.group;
      int s = valid ? r / p.group : 0, gi = valid ? r - s * p.group : 0;
      const char* qp = (const char*)p.q + (((seg_q_row0 + s) * p.heads + kvh * p.group + gi) * D) * 2;
      if constexpr (QK8) {
        // the lane's depth positions are those of the K bytes it reads: head elements [64j + 16g, 64j + 16g + 16), j < NCH
        float f[16 * NCH];
#pragma unroll
        for (int h = 0; h < 2 * NCH; h++) {
          u32x4 z = {0, 0, 0, 0};
          u32x4 raw = valid ? *(const u32x4*)(qp + (64 * (h >> 1) + 16 * g + 8 * (h & 1)) * 2) : z;
          uint32_t w[4] = {raw[0], raw[1], raw[2], raw[3]};
          Unpack<QT, 8>::run(w, f + 8 * h);
        }
        float am = 0.f;
#pragma unroll
        for (int e = 0; e < 16 * NCH; e++) am = fmaxf(am, fabsf(f[e]));
        am = fmaxf(group_max(am), 1e-30f);  // over the four lanes that share the row
        // scale by a power of two that puts the row maximum in [128, 256): element mantissas are untouched, so the
        // eight significant bits of a bf16 element are exactly hi (four) + lo (four)
        const uint32_t be = (__float_as_uint(am) >> 23) & 0xffu;  // biased exponent, >= 27
        const float inv = __uint_as_float((261u - be) << 23);     // 2^(7 - e)
        q_scale[rb] = __uint_as_float((be - 7u) << 23);            // 2^(e - 7)
#pragma unroll
        for (int h = 0; h < NCH; h++) {   // h = which 16 of the lane's positions
          u32x4 hi, lo;
#pragma unroll
          for (int w4 = 0; w4 < 4; w4++) {
            const float* x = f + 16 * h + 4 * w4;
            const float a0 = x[0] * inv, a1 = x[1] * inv, a2 = x[2] * inv, a3 = x[3] * inv;
            const uint32_t wh = pack_fp8x4(a0, a1, a2, a3);
            const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(wh, false), b23 = __builtin_amdgcn_cvt_pk_f32_fp8(wh, true);
            hi[w4] = wh;
            lo[w4] = pack_fp8x4(a0 - b01[0], a1 - b01[1], a2 - b23[0], a3 - b23[1]);
          }
          qreg[rb][h] = hi;        // [0, NCH): hi part
          qreg[rb][NCH + h] = lo;  // [NCH, 2 NCH): lo part
        }
      } else {
#pragma unroll
        for (int j = 0; j < NJ; j++) {
          // head elements this lane contributes to k-step j: 8 consecutive ones, matching the K operand
          int d0 = FP8 ? 64 * (j >> 1) + 16 * g + 8 * (j & 1) : 32 * j + 8 * g;
          u32x4 z = {0, 0, 0, 0};
          qreg[rb][j] = valid ? *(const u32x4*)(qp + d0 * 2) : z;
        }
      }
      limit[rb] = valid ? ((p.causal && p.q_len > 1) ? cu.len - seg_q_len + s + 1 : cu.len) : 0;
      m_run[rb] = kNegFloor;
      l_run[rb] = 0.f;
#pragma unroll
      for (int db = 0; db < NDB; db++) o_acc[rb][db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (p.init_o && cu.j == 0) {
      // Carried state: the segment opens the sequence, so its rows take over the earlier result.  A normalised row O
      // with log-sum-exp L is the state (reference m = L, sum l = 1, accumulator O); the sum is kept in the g == 0
      // lanes because the final sum adds the four lane groups.  L = -inf (no earlier keys) leaves the empty state.
#pragma unroll
      for (int rb = 0; rb < NRB; rb++) {
        int r = rg * (16 * NRB) + rb * 16 + c;
        bool valid = r < seg_q_len * p.group;
        int s = valid ? r / p.group : 0, gi = valid ? r - s * p.group : 0;
        const int64_t orow = (seg_q_row0 + s) * p.heads + kvh * p.group + gi;
        const float l0 = valid ? p.init_lse[orow] : -INFINITY;
        if (l0 != -INFINITY) {
          m_run[rb] = l0;
          l_run[rb] = g == 0 ? 1.f : 0.f;
#pragma unroll
          for (int db = 0; db < NDB; db++) o_acc[rb][db] = *(const f32x4*)(p.init_o + orow * D + 16 * db + 4 * g);
        }
      }
#pragma unroll
      for (int rb = 0; rb < NRB; rb++) {
        asm volatile("" : "+v"(m_run[rb]));
#pragma unroll
        for (int db = 0; db < NDB; db++) asm volatile("" : "+v"(o_acc[rb][db]));  // land here, not in the loop
      }
    }
    // Make the query loads land here: an empty asm that "modifies" each register forces the compiler to put
    // its own vmcnt wait in this (rare) block instead of in the steady-state loop, where such a wait would
    // also wait for every direct-to-LDS load in flight.
#pragma unroll
    for (int rb = 0; rb < NRB; rb++)
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        asm volatile("" : "+v"(qreg[rb][j]));
        // a negative softmax scale is carried by the query (an exact sign flip), so the scale itself is positive
        qreg[rb][j] ^= u32x4{q_sign, q_sign, q_sign, q_sign};
      }
  };

  // SOFF = byte offset of the stage slot inside the wave's LDS ring; a literal at every call site of the
  // single-row-block kernels (folds into the ds_read immediates), a run-time value in the multi-row-block ones
  // The stage body is split in two.  score_step: LDS reads, S^T = K.Q^T, online softmax; leaves V^T operands and
  // packed probabilities in registers and returns whether any row moved its softmax reference (wave-uniform).
  // value_step: O^T += V^T.P^T.  Between them the caller rescales the accumulators when asked to -- outside the
  // steady-state loop, because the accumulators live in accumulation registers that the vector ALU cannot
  // address, and a rescale inside the loop makes the register allocator shuttle all of them on every iteration.
  // With an fp8 cache and several row blocks registers are short: V^T then stays in bytes until the PV product
  // consumes it (widened one 16-column block at a time, in between the MFMAs).
  constexpr bool LATE_V = FP8 && (NRB >= 2 || D == 256);
  // 16-bit cache, head dim 256, ring of eight (two waves per SIMD, 256 registers each): the V^T operands of a tile are
  // 64 registers, as many as the K operands; V^T is read from LDS inside the value step, four 16-column blocks at a
  // time, instead of being held across the softmax, and K in two halves of the head dim.
  constexpr bool LATE_VREAD = !FP8 && D == 256 && SHW == 8;
  // The same ring with an FP8 cache: the 32 registers of V^T bytes are read inside the value step as well, four 16-column
  // blocks at a time, and widened there.
  constexpr bool LATE_VREAD8 = FP8 && D == 256 && SHW == 8;
  // 16-bit rings of two row blocks at head dims up to 128, several tiles per barrier: the K operands of a step's next tile
  // are read from LDS behind this tile's score products (the registers of the operands they replace are free by then), so
  // that they land under the softmax instead of in front of the next tile's first product.
  constexpr bool KPRE = kKPrefetch && !FP8 && NRB == 2 && SH && NS >= 4 && D <= 128 && !LATE_VREAD;
  // Head dim 256 on rings of eight (K read in two halves of the head dim): the first half is carried the same way.
  constexpr bool KPRE2 = kKPrefetch && LATE_VREAD && NRB == 1 && NS >= 4;
  u32x4 k_held[2][KPRE ? NJ : (KPRE2 ? NJ / 2 : 1)];  // the K operands of the tile at hand, carried from tile to tile
  bool have_k_pre = false;
  u32x4 va_op[(LATE_V || LATE_VREAD) ? 1 : NDB];
  i32x2 vraw[(LATE_V && !LATE_VREAD8) ? NDB : 1];
  u32x4 pk[NRB];
  float alpha[NRB];
  // LDS address of a read in ring slot offset SOFF.  Where SOFF is a run-time value (two row blocks: one copy of the tile
  // body for all slots) the slot is added to each distinct lane base once and pinned there, so that the reads of a base
  // differ by immediates only; left to itself the compiler forms (SOFF + constant) per read and spends one vector add on
  // every one of them (24 a tile for a 16-bit cache).  With a constant SOFF everything folds into the immediate anyway.
  auto in_slot = [&](uint32_t base, const uint32_t SOFF) __attribute__((always_inline)) -> uint32_t {
    uint32_t a = base + SOFF;
    if constexpr (NRB != 1 || LATE_VREAD) asm volatile("" : "+v"(a));
    return a;
  };
  auto score_step = [&](const uint32_t SOFF, const Cursor& cu, const uint32_t NEXT_SOFF = 0u, const bool more = false) __attribute__((always_inline)) -> bool {
    const int tok0 = cu.j * kCT;
    // ---- all LDS reads of the stage go out first: 8 K operands, 8 V^T operands (+ scales) ----------------
    u32x4 ka_op[2][NJ];
    f32x4 ksc[2], vsc[2];
    constexpr uint32_t HALF = 16 * G::ROW;  // bytes of one 16-token block of K (or V)
    uint32_t kb[NKA];
#pragma unroll
    for (int i = 0; i < NKA; i++) kb[i] = in_slot(kaddr[i], SOFF);
    if constexpr (!FP8) {
      if constexpr (KPRE) {
        if (!have_k_pre) {
#pragma unroll
          for (int tb = 0; tb < 2; tb++)
#pragma unroll
            for (int j = 0; j < NJ; j++) k_held[tb][j] = *LDS_AT(u32x4, kb[j % NKA] + (tb * HALF + (j / NKA) * (NKA * 64)));
        }
      } else if constexpr (!LATE_VREAD) {
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
          for (int j = 0; j < NJ; j++) ka_op[tb][j] = *LDS_AT(u32x4, kb[j % NKA] + (tb * HALF + (j / NKA) * (NKA * 64)));
      }
      if constexpr (!LATE_VREAD) {
        uint32_t vb[NDB < 8 ? NDB : 8];
#pragma unroll
        for (int i = 0; i < (NDB < 8 ? NDB : 8); i++) vb[i] = in_slot(vaddr[i], SOFF);
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(s16x4, vb[db & 7] + ((db >> 3) * 256)));
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(s16x4, vb[db & 7] + (HALF + (db >> 3) * 256)));
          u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          va_op[db] = u32x4{l2[0], l2[1], h2[0], h2[1]};
        }
      }
    } else {
      u32x4 kraw[2][NJ / 2];
      i32x2 vnow[NDB];
#pragma unroll
      for (int tb = 0; tb < 2; tb++)
#pragma unroll
        for (int jj = 0; jj < NJ / 2; jj++) kraw[tb][jj] = *LDS_AT(u32x4, kb[jj] + (tb * HALF));
      const uint32_t sb = in_slot(saddr, SOFF);
#pragma unroll
      for (int tb = 0; tb < 2; tb++) {
        ksc[tb] = *LDS_AT(f32x4, sb + (64 * tb));
        vsc[tb] = *LDS_AT(f32x4, sb + (128 + 64 * tb));
      }
      if constexpr (!LATE_VREAD8) {
#pragma unroll
        for (int db = 0; db < NDB; db++) vnow[db] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_AT(i32x2, in_slot(vaddr[db], SOFF)));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int tb = 0; tb < 2; tb++)
#pragma unroll
        for (int jj = 0; jj < NJ / 2; jj++) {
          if constexpr (QK8) {  // kept as bytes: [jj] = chunk 4 jj + g of the token row
            ka_op[tb][jj] = kraw[tb][jj];
          } else {
            ka_op[tb][2 * jj] = widen8<QT>(kraw[tb][jj][0], kraw[tb][jj][1]);
            ka_op[tb][2 * jj + 1] = widen8<QT>(kraw[tb][jj][2], kraw[tb][jj][3]);
          }
        }
      if constexpr (!LATE_VREAD8) {
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          if constexpr (LATE_V) vraw[db] = vnow[db];
          else va_op[db] = widen8<QT>((uint32_t)vnow[db][0], (uint32_t)vnow[db][1]);
        }
      }
    }
    if (!FP8) __builtin_amdgcn_sched_barrier(0);
    // ---- S^T = K . Q^T : the two 16-token blocks interleaved so dependent MFMAs are one apart -------------
    f32x4 s_acc[2][NRB];
#pragma unroll
    for (int tb = 0; tb < 2; tb++)
#pragma unroll
      for (int rb = 0; rb < NRB; rb++) s_acc[tb][rb] = f32x4{0.f, 0.f, 0.f, 0.f};
    // Two waves of different workgroups share a SIMD: the one that is feeding the matrix pipe goes first, the other's
    // softmax fills the gaps (FP8 rings: -3 % on the eight-query-token workload; 16-bit rings measured no gain).
    constexpr bool PRIO = SH && FP8;
    if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
    if constexpr (QK8) {
#pragma unroll
      for (int part = 0; part < 2; part++)  // hi, then lo: dependent instructions are 2*NRB apart
#pragma unroll
        for (int h = 0; h < NCH / 2; h++)   // 128 head elements per step
#pragma unroll
          for (int rb = 0; rb < NRB; rb++)
#pragma unroll
            for (int tb = 0; tb < 2; tb++)
              s_acc[tb][rb] = mma_fp8_k128(ka_op[tb][2 * h], ka_op[tb][2 * h + 1], qreg[rb][part * NCH + 2 * h],
                                           qreg[rb][part * NCH + 2 * h + 1], s_acc[tb][rb]);
    } else if constexpr (LATE_VREAD) {
      // the K operands in two halves of the head dim (32 registers each): read, multiply, read, multiply
      auto read_half = [&](int hf, const uint32_t* base, u32x4 (*dst)[KPRE2 ? NJ / 2 : NJ / 2]) __attribute__((always_inline)) {
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
          for (int jj = 0; jj < NJ / 2; jj++) {
            const int j = hf * (NJ / 2) + jj;
            dst[tb][jj] = *LDS_AT(u32x4, base[j % NKA] + (tb * HALF + (j / NKA) * (NKA * 64)));
          }
      };
      if constexpr (KPRE2) {
        u32x4 kh1[2][NJ / 2];
        if (!have_k_pre) read_half(0, kb, k_held);
        read_half(1, kb, kh1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jj = 0; jj < NJ / 2; jj++)
#pragma unroll
          for (int tb = 0; tb < 2; tb++) s_acc[tb][0] = Mma<QT>::run(k_held[tb][jj], qreg[0][jj], s_acc[tb][0]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jj = 0; jj < NJ / 2; jj++)
#pragma unroll
          for (int tb = 0; tb < 2; tb++) s_acc[tb][0] = Mma<QT>::run(kh1[tb][jj], qreg[0][NJ / 2 + jj], s_acc[tb][0]);
        __builtin_amdgcn_sched_barrier(0);
        have_k_pre = more;
        if (have_k_pre) {
          uint32_t kn[NKA];
#pragma unroll
          for (int i = 0; i < NKA; i++) kn[i] = in_slot(kaddr[i], NEXT_SOFF);
          read_half(0, kn, k_held);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
          u32x4 kh[2][NJ / 2];
          read_half(hf, kb, kh);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int jj = 0; jj < NJ / 2; jj++)
#pragma unroll
            for (int rb = 0; rb < NRB; rb++)
#pragma unroll
              for (int tb = 0; tb < 2; tb++) s_acc[tb][rb] = Mma<QT>::run(kh[tb][jj], qreg[rb][hf * (NJ / 2) + jj], s_acc[tb][rb]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int rb = 0; rb < NRB; rb++)
#pragma unroll
          for (int tb = 0; tb < 2; tb++) {
            if constexpr (KPRE) s_acc[tb][rb] = Mma<QT>::run(k_held[tb][j], qreg[rb][j], s_acc[tb][rb]);
            else s_acc[tb][rb] = Mma<QT>::run(ka_op[tb][j], qreg[rb][j], s_acc[tb][rb]);
          }
      if constexpr (KPRE) {
        have_k_pre = more;
        if (have_k_pre) {
          __builtin_amdgcn_sched_barrier(0);  // behind the products above
          uint32_t kn[NKA];
#pragma unroll
          for (int i = 0; i < NKA; i++) kn[i] = in_slot(kaddr[i], NEXT_SOFF);
#pragma unroll
          for (int tb = 0; tb < 2; tb++)
#pragma unroll
            for (int j = 0; j < NJ; j++) k_held[tb][j] = *LDS_AT(u32x4, kn[j % NKA] + (tb * HALF + (j / NKA) * (NKA * 64)));
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
    // ---- online softmax (exp2 domain), lane-local per query row -------------------------------------------
    const bool need_mask = tok0 + kCT > cu.len - qoff;
    const float exp_scale_all = softcap ? 1.0f : p.score_scale;
    bool any_moved = false;
#pragma unroll
    for (int rb = 0; rb < NRB; rb++) {
      // QK8: the scores are those of the query row scaled to absmax 448; its scale goes where the softmax scale goes
      // (kept a positive normal number, so that a masked -inf stays -inf)
      const float exp_scale = QK8 ? (softcap ? 1.0f : fmaxf(exp_scale_all * q_scale[rb], 1e-37f)) : exp_scale_all;
      const float inv_cap_scale = QK8 ? p.inv_cap_scale * q_scale[rb] : p.inv_cap_scale;
      float x[2][4];
#pragma unroll
      for (int tb = 0; tb < 2; tb++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float s = s_acc[tb][rb][i];
          if (FP8) s *= ksc[tb][i];
          x[tb][i] = s;
        }
      // Without softcap the scores stay unscaled here: the (positive) scale sm_scale*log2e commutes with the
      // maximum and is applied inside the exponent as one fused multiply-add per element.
      if (softcap) {
        asm volatile("");  // keeps this a real (wave-uniform) branch: the tanh is too long to compute speculatively
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
          for (int i = 0; i < 4; i++) x[tb][i] = to_logit2<true>(x[tb][i], p.score_scale, p.cap_log2e, inv_cap_scale);
      }
      if (need_mask) {  // only the last tile(s) of a sequence
        int t0 = tok0 + 4 * g;
        asm volatile("" : "+v"(t0));  // the token indices are formed in this block, not ahead of the branch on every tile
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
          for (int i = 0; i < 4; i++)
            if (t0 + 16 * tb + i >= limit[rb]) x[tb][i] = -INFINITY;
      }
      float mt = max2(max3(x[0][0], x[0][1], x[0][2]), max3(x[0][3], x[1][0], max3(x[1][1], x[1][2], x[1][3])));
      mt = group_max(mt) * exp_scale;
      // Lazy rescale: the running reference m_run only moves when the tile maximum exceeds it by more than
      // kRescaleGap (log2 domain).  Probabilities are then at most 2^kRescaleGap instead of 1 -- harmless for
      // fp32 accumulators and 16-bit P -- and because l_run uses the same reference the final O/l is unchanged.
      // After the first tiles of a sequence the accumulator rescale below almost never runs.
      const bool moved = mt > m_run[rb] + kRescaleGap;
      const float m_new = moved ? mt : m_run[rb];
      alpha[rb] = moved ? fast_exp2(m_run[rb] - m_new) : 1.0f;
      m_run[rb] = m_new;
      any_moved |= moved;
      float psum = 0.f;
#pragma unroll
      for (int tb = 0; tb < 2; tb++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float pr = fast_exp2(__builtin_fmaf(x[tb][i], exp_scale, -m_new));
          psum += pr;
          x[tb][i] = FP8 ? pr * vsc[tb][i] : pr;
        }
      l_run[rb] = l_run[rb] * alpha[rb] + psum;
      pk[rb][0] = Mma<QT>::pack(x[0][0], x[0][1]);
      pk[rb][1] = Mma<QT>::pack(x[0][2], x[0][3]);
      pk[rb][2] = Mma<QT>::pack(x[1][0], x[1][1]);
      pk[rb][3] = Mma<QT>::pack(x[1][2], x[1][3]);
    }
    return __any(any_moved);
  };
  auto rescale = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int rb = 0; rb < NRB; rb++)
#pragma unroll
      for (int db = 0; db < NDB; db++) {
        o_acc[rb][db] *= alpha[rb];  // alpha is 1 for rows that kept their reference
        __builtin_amdgcn_sched_barrier(0);  // one tile at a time: keeps the copies out of the accumulation registers short-lived
      }
  };
  auto value_step = [&](const uint32_t SOFF) __attribute__((always_inline)) {
    if constexpr (LATE_VREAD) {
      constexpr uint32_t HALF = 16 * G::ROW;
      constexpr int GB = 4;  // 16-column blocks per round of LDS reads
      uint32_t vb[8];
#pragma unroll
      for (int i = 0; i < 8; i++) vb[i] = in_slot(vaddr[i], SOFF);
      auto read_group = [&](int g0, u32x4* dst) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < GB; e++) {
          const int db = g0 + e;
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(s16x4, vb[db & 7] + ((db >> 3) * 256)));
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(s16x4, vb[db & 7] + (HALF + (db >> 3) * 256)));
          u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          dst[e] = u32x4{l2[0], l2[1], h2[0], h2[1]};
        }
      };
      u32x4 vt[2][GB];
      read_group(0, vt[0]);
#pragma unroll
      for (int gi = 0; gi < NDB / GB; gi++) {
        if (gi + 1 < NDB / GB) read_group((gi + 1) * GB, vt[(gi + 1) & 1]);  // the next round is in flight under this round's products
#pragma unroll
        for (int e = 0; e < GB; e++)
#pragma unroll
          for (int rb = 0; rb < NRB; rb++) o_acc[rb][gi * GB + e] = Mma<QT>::run(vt[gi & 1][e], pk[rb], o_acc[rb][gi * GB + e]);
        __builtin_amdgcn_sched_barrier(0);  // keeps the rounds apart: at most two rounds of operands are live
      }
      return;
    }
    if constexpr (LATE_VREAD8) {
      constexpr int GB = 4;
      auto read_group = [&](int g0, i32x2* dst) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < GB; e++) dst[e] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_AT(i32x2, vaddr[g0 + e] + SOFF));
      };
      i32x2 vr[2][GB];
      read_group(0, vr[0]);
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int gi = 0; gi < NDB / GB; gi++) {
        if (gi + 1 < NDB / GB) read_group((gi + 1) * GB, vr[(gi + 1) & 1]);
#pragma unroll
        for (int e = 0; e < GB; e++) {
          const u32x4 vt = widen8<QT>((uint32_t)vr[gi & 1][e][0], (uint32_t)vr[gi & 1][e][1]);
#pragma unroll
          for (int rb = 0; rb < NRB; rb++) o_acc[rb][gi * GB + e] = Mma<QT>::run(vt, pk[rb], o_acc[rb][gi * GB + e]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_setprio(0);
      return;
    }
    if constexpr (SH && FP8) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int db = 0; db < NDB; db++) {
      u32x4 vt;
      if constexpr (LATE_V) vt = widen8<QT>((uint32_t)vraw[db][0], (uint32_t)vraw[db][1]);
      else vt = va_op[db];
#pragma unroll
      for (int rb = 0; rb < NRB; rb++) o_acc[rb][db] = Mma<QT>::run(vt, pk[rb], o_acc[rb][db]);
    }
    if constexpr (SH && FP8) __builtin_amdgcn_s_setprio(0);
  };

  auto end_segment = [&](const Cursor& cu, bool complete, int which) __attribute__((always_inline)) {
#pragma unroll
    for (int rb = 0; rb < NRB; rb++) {
      int r = rg * (16 * NRB) + rb * 16 + c;
      float l_tot = group_sum(l_run[rb]);
      float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
      if (r >= seg_q_len * p.group) continue;
      if (complete) {
        int s = r / p.group, gi = r - s * p.group;
        const int64_t orow = (seg_q_row0 + s) * p.heads + kvh * p.group + gi;
        if (p.final_o) {  // fp32 rows + LSE for a later merge with another call
#pragma unroll
          for (int db = 0; db < NDB; db++) *(f32x4*)(p.final_o + orow * D + 16 * db + 4 * g) = o_acc[rb][db] * inv;
          if (g == 0) p.final_lse[orow] = l_tot > 0.f ? m_run[rb] + log2f(l_tot) : -INFINITY;
          continue;
        }
        uint16_t* op = (uint16_t*)p.out + orow * D;
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          f32x4 o = o_acc[rb][db] * inv;
          u32x2 w;
          w[0] = Mma<QT>::pack(o[0], o[1]);
          w[1] = Mma<QT>::pack(o[2], o[3]);
          *(u32x2*)(op + 16 * db + 4 * g) = w;
        }
      } else {
        int64_t grow = ((int64_t)(2 * part + which) * p.heads_kv + kvh) * p.rows + r;
        if (p.part16) {
          uint16_t* pp = (uint16_t*)p.part_o + grow * D;
#pragma unroll
          for (int db = 0; db < NDB; db++) {
            f32x4 o = o_acc[rb][db] * inv;
            u32x2 w;
            w[0] = Mma<QT>::pack(o[0], o[1]);
            w[1] = Mma<QT>::pack(o[2], o[3]);
            *(u32x2*)(pp + 16 * db + 4 * g) = w;
          }
        } else {
          float* pp = p.part_o + grow * D;
#pragma unroll
          for (int db = 0; db < NDB; db++) *(f32x4*)(pp + 16 * db + 4 * g) = o_acc[rb][db] * inv;
        }
        if (g == 0) p.part_lse[grow] = l_tot > 0.f ? m_run[rb] + log2f(l_tot) : -INFINITY;
      }
    }
  };

  // ---- software pipeline over this wave's tiles: stage u lives in LDS slot u % NS -------------------------
  // Outer loop = segments (maximal runs of tiles of one sequence inside this wave's range), inner loop = the
  // tiles of a segment.  The accumulators are initialised in the inner loop's preheader and stay in their
  // registers across it; issuing runs NS-1 tiles ahead of consumption and is oblivious to segment borders.
  Cursor ci = start, cc = start;
  uint32_t ci_row = ps16 ? 0u : locate(ci);  // pool row of the tile at ci
  int issued = 0;
  auto advance = [&]() __attribute__((always_inline)) {  // ci to the next tile of the range (there is one)
    cursor_next(ci, p, ps16);
    if (ps16) return;
    if (ci.j == 0 || (paged && ci.off == 0)) ci_row = locate(ci);
    else ci_row += kCT;
  };
  for (; issued < NS - 1 && issued < n_units;) {
    issue(ci, issued, ci_row);
    if (++issued < n_units) advance();
  }
  auto issue_ahead = [&](int ring) __attribute__((always_inline)) {
    if (issued < n_units) {
      issue(ci, ring == 0 ? NS - 1 : ring - 1, ci_row);  // the ring slot consumed in the previous iteration
      if (++issued < n_units) advance();
    }
  };
  auto wait_stage = [&](int u) __attribute__((always_inline)) {
    const int ahead = issued - u - 1;  // stages issued after the one consumed now
    if (ahead >= 3) wait_vmcnt<(NS > 3 ? 3 : NS - 1) * IPSW>();
    else if (ahead == 2) wait_vmcnt<(NS > 2 ? 2 : NS - 1) * IPSW>();
    else if (ahead == 1) wait_vmcnt<IPSW>();
    else wait_vmcnt<0>();
  };
  auto run_score_step = [&](int ring) __attribute__((always_inline)) -> bool {
    if constexpr (NRB == 1) {
      // one copy of the body per ring slot: the slot offset folds into the LDS read immediates
      if (ring == 0) return score_step(0u, cc);
      else if (NS > 1 && ring == 1) return score_step((uint32_t)G::STAGE, cc);
      else if (NS > 2 && ring == 2) return score_step(2u * G::STAGE, cc);
      else return score_step(3u * G::STAGE, cc);
    } else {
      return score_step((uint32_t)ring * G::STAGE, cc);  // large body: a single copy keeps the kernel in the instruction cache
    }
  };
  auto run_score_step_pre = [&](int ring, bool more) __attribute__((always_inline)) -> bool {  // more: the step has another tile
    // (one copy of the body with a run-time slot offset, also for one row block: with the operands carried across four
    // copies the compiler spills)
    return score_step((uint32_t)ring * G::STAGE, cc, (uint32_t)((ring + 1) & (NS - 1)) * G::STAGE, more);
  };
  int u = 0, ring = 0, seg_count = 0;
  // two waves per SIMD: the accumulators are ordinary vector registers, the rescale can sit in the loop
  constexpr bool RESCALE_IN_LOOP = (SH && (D <= 128 || SHW == 8)) || (FP8 && NRB == 2);
  constexpr bool PAIRS = kPairSteps && SH && NS >= 4 && RESCALE_IN_LOOP;
  // A fetch instruction holds its wave while the compute unit's address path takes it.  Where a wave issues four or more
  // of them per stage (head dim 256; fp8 and 64-byte-row rings of two) a step's second fetch goes out between the step's
  // tiles instead of in one burst with the first: 8 x 1024-token chunks at head dim 256 on 32 K prefixes 12.28 ms with the
  // burst, 11.54 with one tile per barrier, 10.92 this way; the eight-query-token fp8 configuration 152.9 -> 150.8 us.
  // With two instructions per stage and two tiles per step (16-bit rings of eight at head dim 128 on four stages) the burst
  // was the faster by 1 %; on eight stages, four tiles per step, spreading wins again (413 -> 406 us).
  constexpr bool SPLIT_ISSUE = IPSW >= 4 || NS == 8;
  constexpr int STEP = PAIRS ? NS / 2 : 1;  // tiles per barrier: half the ring is read while the other half is refilled
  while (u < n_units) {
    const int seg_first_j = cc.j;
    const int seg_units = min(cc.nt - cc.j, n_units - u);
    if (!LATE) issue_ahead(ring);  // before the query loads, so the next tile is already in flight while they land
    begin_segment(cc);
    int k = 0;
    if constexpr (PAIRS) {
      while (k < seg_units) {
        const int step = min(STEP, seg_units - k);  // tiles of this step: u .. u + step - 1, in ring slots u % NS and on
        wait_stage(u + step - 1);                    // the later tile has landed, so has the earlier (requests complete in order)
        // Past the barrier every wave's part of both tiles is in LDS, and every wave has finished reading the tiles before
        // u: their slots may be refilled.  Tile t goes to slot t % NS, so the request may run up to tile u + NS - 1.
        asm volatile("s_barrier" ::: "memory");
        const int u_step = u;
        auto issue_one = [&]() __attribute__((always_inline)) {
          if (issued < n_units && issued - NS < u_step) {
            issue(ci, issued & (NS - 1), ci_row);
            if (++issued < n_units) advance();
          }
        };
        if constexpr (SPLIT_ISSUE) {
          issue_one();
        } else {
          while (issued < n_units && issued - NS < u_step) issue_one();
        }
#pragma nounroll
        for (int sub = 0; sub < step; ++sub) {  // (a loop, not two copies: the body is large)
          bool moved_;
          if constexpr (KPRE || KPRE2) moved_ = run_score_step_pre(ring, sub + 1 < step);
          else moved_ = run_score_step(ring);
          if (__builtin_expect(moved_, 0)) rescale();
          value_step((uint32_t)ring * G::STAGE);
          ++u;
          ++cc.j;
          ring = (ring + 1) & (NS - 1);
          ++k;
          if constexpr (SPLIT_ISSUE) issue_one();
        }
        if constexpr (SPLIT_ISSUE) {
          while (issued < n_units && issued - NS < u_step) issue_one();  // (a step of one tile may have two slots to refill)
        }
      }
    }
    while (!PAIRS && k < seg_units) {
      bool moved = false;
      for (; k < seg_units; ++k) {  // steady state: no tile in here rescales the accumulators
        if (!LATE && k > 0) issue_ahead(ring);
        wait_stage(u);
        if (SH) {
          // Own part of tile u has landed; past the barrier so have the others', and every wave of the workgroup
          // has finished reading tile u-1, whose slot the next fetch overwrites.
          asm volatile("s_barrier" ::: "memory");
        }
        if (LATE) issue_ahead(ring);
        moved = run_score_step(ring);
        if constexpr (RESCALE_IN_LOOP) {
          if (__builtin_expect(moved, 0)) rescale();
          moved = false;
        } else {
          if (__builtin_expect(moved, 0)) break;
        }
        value_step((uint32_t)ring * G::STAGE);
        ++u;
        ++cc.j;
        ring = ring + 1 == NS ? 0 : ring + 1;
      }
      if (moved) {  // rare after the first tiles of a sequence: finish this tile out of line, then re-enter
        rescale();
        value_step((uint32_t)ring * G::STAGE);
        ++u;
        ++cc.j;
        ring = ring + 1 == NS ? 0 : ring + 1;
        ++k;
      }
    }
    --cc.j;  // end_segment and cursor_next see the last tile of the segment
    end_segment(cc, seg_first_j == 0 && cc.j == cc.nt - 1, seg_count == 0 ? 0 : 1);
    ++seg_count;
    cursor_next(cc, p, ps16);
  }
}

// Merge the partials of sequences that span more than one partition, and zero-fill empty sequences.
//   lse = log2 sum_s 2^(lse_s - max) + max ; O = sum_s 2^(lse_s - lse) * O_s   (reference combine,
//   src/tileops/kernels/attention/gqa_decode_paged.py:344-374), on fp32 or 16-bit partial rows (DecodeParams::part16) and fp32 log-sum-exps.
// Four waves work on one (sequence, kv head, query row) at a time.  Every wave forms the maximum and the sum of
// weights over all partitions of the sequence (lane i fetches the LSE of partition i, two wave reductions per 64);
// the weighted sum of the partial rows is split over the waves (wave w takes partitions w, w+4, ...), eight
// independent row loads in flight per wave, every lane two head elements; the four sums meet in LDS.  With at
// most eight partitions wave 0 works alone and the others leave at once.  A single
// sequence spread over hundreds of partitions (batch-1 long-context decode) is then merged in a few load round
// trips instead of one per partition.  64*kCombineWaves threads; the launcher takes the one-wave instance when the
// average sequence spans at most eight partitions.
// One lane's two elements of a partial output row: fp32, or the query's 16-bit type widened.
template <typename QT>
__device__ __forceinline__ f32x2 load_part2(const DecodeParams& p, int64_t slot, int hd, int dl) {
  if (p.part16) return unpack2<QT>(*(const uint32_t*)((const uint16_t*)p.part_o + slot * hd + dl));
  return *(const f32x2*)(p.part_o + slot * hd + dl);
}
// The same load with the 16-bit pair left as bits in element 0 (many loads in flight, widened when consumed).
__device__ __forceinline__ f32x2 load_part2_raw(const DecodeParams& p, int64_t slot, int hd, int dl) {
  if (p.part16) return f32x2{__builtin_bit_cast(float, *(const uint32_t*)((const uint16_t*)p.part_o + slot * hd + dl)), 0.f};
  return *(const f32x2*)(p.part_o + slot * hd + dl);
}

template <typename QT, int kCombineWaves>
__device__ __forceinline__ void combine_row(const DecodeParams& p, const int* __restrict__ ws_prefix, f32x2 (*red)[64], int b, int row_all, int4 rec,
                                            int wave);
template <typename QT, int R>
__device__ __forceinline__ void combine_rows_at_once(const DecodeParams& p, int b, int row0, int row_end, int4 rec);

// grid (ceil(heads_kv*rows / rows_per_wg), batch, halves of a 256-wide head): a workgroup takes rows_per_wg consecutive
// rows of one sequence.  With thousands of rows per sequence (prefill chunks) most sequences lie inside one partition
// and need no merge at all: the workgroup reads the sequence's record once and leaves, instead of one workgroup per row
// doing so (131 072 of them took 28 us on an 8 x 512-row call).
template <typename QT, int kCombineWaves, bool kManyRows = false>
__global__ __launch_bounds__(256) void paged_decode_mfma_combine_kernel(const DecodeParams p, const int* __restrict__ ws_prefix, int rows_per_wg) {
  // always four waves: either they share one row at a time (kCombineWaves == 4) or each takes every fourth row of the
  // workgroup's range on its own (kCombineWaves == 1)
  static_assert(kCombineWaves == 1 || kCombineWaves == 4, "one or four waves per row");
  __shared__ f32x2 red[kCombineWaves][64];
  const int b = blockIdx.y;
  const int4 rec = ((const int4*)ws_prefix)[b];  // the only load everything else depends on
  if (rec.y >= 0 && rec.y == rec.z) return;  // one wave covered the whole sequence and wrote the output itself
  const int row_end = min((int)(blockIdx.x + 1) * rows_per_wg, p.heads_kv * p.rows);
  const int phys_wave = uni(threadIdx.x >> 6);
  if constexpr (kCombineWaves == 1) {
    constexpr int R = 4;
    if (kManyRows && rows_per_wg >= 4 * R && rec.y >= 0 && rec.z - rec.y < 8 && (rec.w & 2) == 0) {
      // many rows per workgroup, at most eight partials each: a wave takes R rows and has the loads of all of them in flight together
      for (int row0 = blockIdx.x * rows_per_wg + phys_wave * R; row0 < row_end; row0 += 4 * R) combine_rows_at_once<QT, R>(p, b, row0, row_end, rec);
      return;
    }
    for (int row_all = blockIdx.x * rows_per_wg + phys_wave; row_all < row_end; row_all += 4)
      combine_row<QT, 1>(p, ws_prefix, red, b, row_all, rec, 0);
  } else {
    for (int row_all = blockIdx.x * rows_per_wg; row_all < row_end; row_all++) {
      combine_row<QT, kCombineWaves>(p, ws_prefix, red, b, row_all, rec, phys_wave);
      if (row_all + 1 < row_end) __syncthreads();  // red[] is reused by the next row
    }
  }
}

template <typename QT, int kCombineWaves>
__device__ __forceinline__ void combine_row(const DecodeParams& p, const int* __restrict__ ws_prefix, f32x2 (*red)[64], int b, int row_all, int4 rec,
                                            int wave) {  // wave = this wave's index among the kCombineWaves that share the row
  const int lane = threadIdx.x & 63;
  const int kvh = row_all / p.rows, r = row_all - kvh * p.rows;
  const int s = r / p.group, gi = r - s * p.group;
  if (p.cu_q && r >= q_len_of(p, b) * p.group) return;  // packed queries: this sequence has fewer rows
  const int64_t orow = (q_row0_of(p, b) + s) * p.heads + kvh * p.group + gi;
  // every lane owns two head elements of the 128 this workgroup merges (blockIdx.z picks the half of a 256-wide
  // head); with head dim 64 the upper half of the wave idles (reads element 0, stores nothing)
  const int hd = p.dim;
  const bool owns = 2 * lane < hd;
  const int dl = owns ? 2 * lane + 128 * (int)blockIdx.z : 0;
  uint32_t* op = (uint32_t*)((uint16_t*)p.out + orow * hd) + (dl >> 1);
  auto store = [&](float a0, float a1, float lse) {
    if (!owns) return;
    if (p.final_o) {
      *(f32x2*)(p.final_o + orow * hd + dl) = f32x2{a0, a1};
      if (lane == 0 && blockIdx.z == 0) p.final_lse[orow] = lse;
    } else {
      *op = Mma<QT>::pack(a0, a1);
    }
  };
  const int p_first = rec.y, p_last = rec.z;
  if (p_first < 0) {  // empty sequence: the attention kernel never visits it
    if (wave == 0) store(0.f, 0.f, -INFINITY);
    return;
  }
  const bool gaps = (rec.w & 2) != 0, first_in_slot1 = (rec.w & 1) != 0;
  const int64_t NP = p.n_parts;
  const int64_t T = gaps ? ((const int4*)ws_prefix)[p.batch].x : 0;
  const int64_t rows_all = (int64_t)p.heads_kv * p.rows;
  const int n = p_last - p_first + 1;
  auto slot_of = [&](int pp) { return (int64_t)(2 * pp + ((pp == p_first && first_in_slot1) ? 1 : 0)) * rows_all + row_all; };
  auto owns_tiles = [&](int pp) { return !gaps || part_begin(pp + 1, T, NP) > part_begin(pp, T, NP); };
  constexpr int PRE = 8;
  // up to eight partitions (the usual case when many sequences share the chip): one wave does it all
  const int nw = n <= PRE ? 1 : kCombineWaves;
  if (wave >= nw) return;
  // this wave's first eight partial rows go out together with the LSEs, before any weight is known
  f32x2 rows[PRE];
#pragma unroll
  for (int i = 0; i < PRE; i++) rows[i] = load_part2<QT>(p, slot_of(min(p_first + wave + nw * i, p_last)), hd, dl);
  // lane i keeps the LSE of partition i of the first 64 (all of them, as a rule); further ones are re-read
  const float lse0 = (p_first + lane <= p_last && owns_tiles(p_first + lane)) ? p.part_lse[slot_of(p_first + lane)] : -INFINITY;
  float M = lse0;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) M = fmaxf(M, __shfl_xor(M, m, 64));
  for (int base = 64; base < n; base += 64) {
    const int pp = p_first + base + lane;
    float lse = (pp <= p_last && owns_tiles(pp)) ? p.part_lse[slot_of(pp)] : -INFINITY;
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) lse = fmaxf(lse, __shfl_xor(lse, m, 64));
    M = fmaxf(M, lse);
  }
  const float w0 = (M != -INFINITY && lse0 != -INFINITY) ? fast_exp2(lse0 - M) : 0.f;  // weight of partition `lane`
  float W = w0;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) W += __shfl_xor(W, m, 64);
  if (M != -INFINITY) {
    for (int base = 64; base < n; base += 64) {  // second pass over the (now cached) LSEs
      const int pp = p_first + base + lane;
      float w = (pp <= p_last && owns_tiles(pp)) ? fast_exp2(p.part_lse[slot_of(pp)] - M) : 0.f;
#pragma unroll
      for (int m = 1; m < 64; m <<= 1) w += __shfl_xor(w, m, 64);
      W += w;
    }
  }
  float acc0 = 0.f, acc1 = 0.f;
  if (W > 0.f) {
    for (int i0 = 0; wave + nw * i0 < n; i0 += PRE) {
      float wt[PRE];
#pragma unroll
      for (int i = 0; i < PRE; i++) {
        const int idx = wave + nw * (i0 + i), pp = p_first + idx;  // wave-uniform
        if (idx < 64) wt[i] = __shfl(w0, idx, 64);
        else wt[i] = (pp <= p_last && owns_tiles(pp)) ? fast_exp2(p.part_lse[slot_of(pp)] - M) : 0.f;
        if (i0 > 0) rows[i] = load_part2<QT>(p, slot_of(min(pp, p_last)), hd, dl);
      }
#pragma unroll
      for (int i = 0; i < PRE; i++)
        if (wt[i] != 0.f) {  // an unwritten slot may hold anything, NaN included
          acc0 = fmaf(wt[i], rows[i][0], acc0);
          acc1 = fmaf(wt[i], rows[i][1], acc1);
        }
    }
  }
  if (nw > 1) {  // uniform over the workgroup: either every wave is here or only wave 0 exists
    red[wave][lane] = f32x2{acc0, acc1};
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 1; w < kCombineWaves; w++) {
      acc0 += red[w][lane][0];
      acc1 += red[w][lane][1];
    }
  }
  const float inv = W > 0.f ? 1.0f / W : 0.f;
  store(acc0 * inv, acc1 * inv, W > 0.f ? M + log2f(W) : -INFINITY);
}

template <typename QT, int R, bool P16>
__device__ __forceinline__ void combine_rows_at_once_t(const DecodeParams& p, int b, int row0, int row_end, int4 rec) {
  constexpr int PRE = 8;
  constexpr int ES = P16 ? 2 : 4;  // bytes per element of a partial row
  const int lane = threadIdx.x & 63;
  const int hd = p.dim;
  const bool owns = 2 * lane < hd;
  const int dl = owns ? 2 * lane + 128 * (int)blockIdx.z : 0;
  const int p_first = rec.y, p_last = rec.z, n = p_last - p_first + 1;
  const bool first_in_slot1 = (rec.w & 1) != 0;
  const int64_t rows_all = (int64_t)p.heads_kv * p.rows;
  const int q_rows = p.cu_q ? q_len_of(p, b) * p.group : p.rows;
  // Addresses: partition i's copy of row row0 is formed once (wave-uniform, 64-bit); the wave's other rows lie whole rows
  // behind it, and a lane adds its two elements' offset.  (Formed per load, the 64-bit products were 2000 scalar
  // instructions a wave -- the kernel was bound by them.)
  const uint32_t row_bytes = (uint32_t)hd * ES, lane_off = (uint32_t)dl * ES;
  const char* base[PRE];
#pragma unroll
  for (int i = 0; i < PRE; i++) {
    const int pp = min(p_first + i, p_last);
    const int64_t slot = (int64_t)(2 * pp + ((pp == p_first && first_in_slot1) ? 1 : 0)) * rows_all + row0;
    base[i] = uni_ptr((const char*)p.part_o + slot * (int64_t)row_bytes);
  }
  const int lp = min(p_first + lane, p_last);
  const float* lse_lane = p.part_lse + ((int64_t)(2 * lp + ((lp == p_first && first_in_slot1) ? 1 : 0)) * rows_all + row0);
  const int last_r = row_end - 1 - row0;  // rows past the workgroup's range re-read its last row and are not stored
  uint32_t raw[R][PRE][P16 ? 1 : 2];
  float lse[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    const uint32_t roff = (uint32_t)min(r, last_r) * row_bytes + lane_off;
#pragma unroll
    for (int i = 0; i < PRE; i++) {
      if constexpr (P16) {
        raw[r][i][0] = *(const uint32_t*)(base[i] + roff);
      } else {
        const u32x2 w = *(const u32x2*)(base[i] + roff);
        raw[r][i][0] = w[0];
        raw[r][i][1] = w[1];
      }
    }
    lse[r] = lane < n ? lse_lane[min(r, last_r)] : -INFINITY;
  }
  // row indices of row0, stepped from row to row (divisions cost more than everything else a row needs)
  int kvh = row0 / p.rows, rr = row0 - kvh * p.rows, s = rr / p.group, gi = rr - s * p.group;
  const int64_t q_row0 = q_row0_of(p, b);
#pragma unroll
  for (int r = 0; r < R; r++) {
    const bool live = r <= last_r && rr < q_rows;  // (packed queries: this sequence may have fewer rows)
    const int64_t orow = (q_row0 + s) * p.heads + kvh * p.group + gi;
    if (++gi == p.group) {
      gi = 0;
      ++s;
    }
    if (++rr == p.rows) {
      rr = 0;
      s = 0;
      gi = 0;
      ++kvh;
    }
    if (!live) continue;
    // the first eight lanes hold the log-sum-exps: as wave-uniform values, so that nothing below crosses lanes
    float l[PRE], M = -INFINITY;
#pragma unroll
    for (int i = 0; i < PRE; i++) {
      l[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, lse[r]), i));
      M = fmaxf(M, l[i]);
    }
    float W = 0.f, acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < PRE; i++) {
      const float wt = (M != -INFINITY && l[i] != -INFINITY) ? fast_exp2(l[i] - M) : 0.f;
      W += wt;
      f32x2 row;
      if constexpr (P16) row = unpack2<QT>(raw[r][i][0]);
      else row = f32x2{__builtin_bit_cast(float, raw[r][i][0]), __builtin_bit_cast(float, raw[r][i][1])};
      if (wt != 0.f) {  // an unwritten slot may hold anything, NaN included
        acc0 = fmaf(wt, row[0], acc0);
        acc1 = fmaf(wt, row[1], acc1);
      }
    }
    const float inv = W > 0.f ? 1.0f / W : 0.f;
    if (!owns) continue;
    if (p.final_o) {
      *(f32x2*)(p.final_o + orow * hd + dl) = f32x2{acc0 * inv, acc1 * inv};
      if (lane == 0 && blockIdx.z == 0) p.final_lse[orow] = W > 0.f ? M + log2f(W) : -INFINITY;
    } else {
      *((uint32_t*)((uint16_t*)p.out + orow * hd) + (dl >> 1)) = Mma<QT>::pack(acc0 * inv, acc1 * inv);
    }
  }
}

// R rows of one sequence merged by one wave, every load of every row issued before the first is consumed: with tens of
// thousands of rows (eight query tokens x group 8 x 32 sequences) the merge kernel is otherwise two rounds of workgroups,
// each a chain of three dependent reads.  At most eight partials per row, every partition owning tiles (the caller checks).
template <typename QT, int R>
__device__ __forceinline__ void combine_rows_at_once(const DecodeParams& p, int b, int row0, int row_end, int4 rec) {
  if (p.part16) combine_rows_at_once_t<QT, R, true>(p, b, row0, row_end, rec);
  else combine_rows_at_once_t<QT, R, false>(p, b, row0, row_end, rec);
}

// The same merge for calls whose sequences span very many partitions each (batch-1 long-context decode).
// The waves of a workgroup work on one (sequence, kv head, query row) at a time.  A lane owns four consecutive head
// elements, so 32 lanes (16 at head dim 64) cover a partial row and the two (four) lane groups of a wave take different
// partitions with one 16-byte load each.  Every wave first fetches up to four LSEs per lane (the first 256 partitions,
// one round trip), forms the maximum and the sum of weights, and meanwhile has its first eight row loads in flight;
// the weighted sums of the groups meet through lane shuffles, those of the waves in LDS.  With 16 waves a sequence
// spread over 256 partitions (batch-1 long-context decode) is merged in one round of loads.  When fewer tiles than
// partitions exist, only the partitions that own a tile (one each) are visited.
constexpr int kCombinePre = 8;   // row loads in flight per wave
constexpr int kCombineLse = 4;   // LSEs kept per lane (first 64 * 4 partitions of the sequence)

template <typename QT, int kCombineWaves>
__device__ __forceinline__ void combine_row_wide(const DecodeParams& p, const int* __restrict__ ws_prefix, f32x4 (*red)[64], int b, int row_all, int4 rec) {
  const int lane = threadIdx.x & 63, wave = uni(threadIdx.x >> 6);
  const int kvh = row_all / p.rows, r = row_all - kvh * p.rows;
  const int s = r / p.group, gi = r - s * p.group;
  if (p.cu_q && r >= q_len_of(p, b) * p.group) return;  // packed queries: this sequence has fewer rows
  const int64_t orow = (q_row0_of(p, b) + s) * p.heads + kvh * p.group + gi;
  const int hd = p.dim;
  const int lpp = (hd < 128 ? hd : 128) >> 2;     // lanes per partial row (blockIdx.z picks the half of a 256-wide head)
  const int ngrp = 64 / lpp, grp = lane / lpp;    // lane groups of a wave: each takes its own partition
  const int dl = 4 * (lane - grp * lpp) + 128 * (int)blockIdx.z;
  auto store = [&](f32x4 a, float lse) {
    if (grp != 0) return;
    if (p.final_o) {
      *(f32x4*)(p.final_o + orow * hd + dl) = a;
      if (lane == 0 && blockIdx.z == 0) p.final_lse[orow] = lse;
    } else {
      u32x2 w;
      w[0] = Mma<QT>::pack(a[0], a[1]);
      w[1] = Mma<QT>::pack(a[2], a[3]);
      *(u32x2*)((uint16_t*)p.out + orow * hd + dl) = w;
    }
  };
  const int p_first = rec.y, p_last = rec.z;
  if (p_first < 0) {  // empty sequence: the attention kernel never visits it
    if (wave == 0) store(f32x4{0.f, 0.f, 0.f, 0.f}, -INFINITY);
    return;
  }
  const bool gaps = (rec.w & 2) != 0, first_in_slot1 = (rec.w & 1) != 0;  // (rec is wave-uniform: see the caller)
  const int64_t rows_all = (int64_t)p.heads_kv * p.rows;
  // fewer tiles than partitions: the sequence's tiles sit one to a partition, the partitions in between own nothing;
  // tile t then belongs to partition ((t + 1) * n_parts - 1) / T, and (t + 1) * n_parts stays far below 2^31
  const uint32_t T = gaps ? (uint32_t)uni(((const int4*)ws_prefix)[p.batch].x) : 1u, NP = (uint32_t)p.n_parts;
  const int n = gaps ? uni(((const int4*)ws_prefix)[b + 1].x) - rec.x : p_last - p_first + 1;
  auto slot_at = [&](int i) {
    const int ii = i < n ? i : n - 1;
    int pp = p_first + ii;
    if (gaps) pp = (int)(((uint32_t)(rec.x + ii + 1) * NP - 1u) / T);
    return (int64_t)(2 * pp + ((pp == p_first && first_in_slot1) ? 1 : 0)) * rows_all + row_all;
  };
  constexpr int PRE = kCombinePre, KL = kCombineLse;
  // few partitions (the usual case when many sequences share the chip): one wave does it all
  const int nw = n <= PRE * ngrp ? 1 : kCombineWaves;
  if (wave >= nw) return;
  // this wave's first row loads go out together with the LSEs, before any weight is known; load j of wave w covers
  // partitions (j*nw + w)*ngrp .. +ngrp-1 of the sequence, one per lane group
  f32x4 rows[PRE];
#pragma unroll
  for (int i = 0; i < PRE; i++) rows[i] = *(const f32x4*)(p.part_o + slot_at((i * nw + wave) * ngrp + grp) * hd + dl);
  float lse[KL];
#pragma unroll
  for (int k = 0; k < KL; k++) lse[k] = 64 * k + lane < n ? p.part_lse[slot_at(64 * k + lane)] : -INFINITY;
  float M = fmaxf(fmaxf(lse[0], lse[1]), fmaxf(lse[2], lse[3]));
  static_assert(KL == 4, "four LSEs per lane");
  for (int base = 64 * KL; base < n; base += 64) M = fmaxf(M, base + lane < n ? p.part_lse[slot_at(base + lane)] : -INFINITY);
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) M = fmaxf(M, __shfl_xor(M, m, 64));
  float wk[KL], W = 0.f;
#pragma unroll
  for (int k = 0; k < KL; k++) {
    wk[k] = (M != -INFINITY && lse[k] != -INFINITY) ? fast_exp2(lse[k] - M) : 0.f;  // weight of partition 64k + lane
    W += wk[k];
  }
  if (M != -INFINITY)
    for (int base = 64 * KL; base < n; base += 64) W += base + lane < n ? fast_exp2(p.part_lse[slot_at(base + lane)] - M) : 0.f;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) W += __shfl_xor(W, m, 64);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (W > 0.f) {
    for (int j0 = 0; (j0 * nw + wave) * ngrp < n; j0 += PRE) {
      float wt[PRE];
#pragma unroll
      for (int i = 0; i < PRE; i++) {
        const int base = ((j0 + i) * nw + wave) * ngrp, idx = base + grp;  // base is wave-uniform and a multiple of ngrp
        if (base < 64 * KL) {
          const int k = base >> 6;
          const float src = k == 0 ? wk[0] : (k == 1 ? wk[1] : (k == 2 ? wk[2] : wk[3]));
          wt[i] = __shfl(src, idx & 63, 64);  // (0 for indices past the last partition)
        } else {
          wt[i] = idx < n ? fast_exp2(p.part_lse[slot_at(idx)] - M) : 0.f;
        }
        if (j0 > 0) rows[i] = *(const f32x4*)(p.part_o + slot_at(idx) * hd + dl);
      }
#pragma unroll
      for (int i = 0; i < PRE; i++)
        if (wt[i] != 0.f) acc += wt[i] * rows[i];  // an unwritten slot may hold anything, NaN included
    }
  }
  // the lane groups of the wave, then the waves
  if (ngrp == 4) {
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] += __shfl_xor(acc[e], 16, 64);
  }
#pragma unroll
  for (int e = 0; e < 4; e++) acc[e] += __shfl_xor(acc[e], 32, 64);
  if (nw > 1) {  // uniform over the workgroup: either every wave is here or only wave 0 exists
    red[wave][lane] = acc;
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 1; w < kCombineWaves; w++) acc += red[w][lane];
  }
  const float inv = W > 0.f ? 1.0f / W : 0.f;
  store(acc * inv, W > 0.f ? M + log2f(W) : -INFINITY);
}

// grid (ceil(heads_kv*rows / rows_per_wg), batch, halves of a 256-wide head): a workgroup takes rows_per_wg consecutive
// rows of one sequence.  With thousands of rows per sequence (prefill chunks) most sequences lie inside one partition
// and need no merge at all: the workgroup reads the sequence's record once and leaves, instead of one workgroup per row
// doing so (131 072 of them took 28 us on an 8 x 512-row call).
template <typename QT, int kCombineWaves>
__global__ __launch_bounds__(64 * kCombineWaves) void paged_decode_mfma_combine_wide_kernel(const DecodeParams p, const int* __restrict__ ws_prefix,
                                                                                       int rows_per_wg) {
  __shared__ f32x4 red[kCombineWaves][64];
  const int b = blockIdx.y;
  const int4 recv = ((const int4*)ws_prefix)[b];  // the only load everything else depends on
  const int4 rec = {uni(recv.x), uni(recv.y), uni(recv.z), uni(recv.w)};  // scalar: every branch on it is a scalar branch
  if (rec.y >= 0 && rec.y == rec.z) return;  // one wave covered the whole sequence and wrote the output itself
  const int row_end = min((int)(blockIdx.x + 1) * rows_per_wg, p.heads_kv * p.rows);
  for (int row_all = blockIdx.x * rows_per_wg; row_all < row_end; row_all++) {
    combine_row_wide<QT, kCombineWaves>(p, ws_prefix, red, b, row_all, rec);
    if (kCombineWaves > 1 && row_all + 1 < row_end) __syncthreads();  // red[] is reused by the next row
  }
}

// Unshared waves per workgroup: with a 16-bit cache a stage is 16 KiB, two stages x four waves fill the LDS of a CU.  With an
// fp8 cache a stage is half that, so eight waves fit: the eight kv heads of a page set then sit in one CU and the
// 32-byte sectors of the scale rows (all heads of a token) are fetched once instead of once per workgroup.

template <typename QT, typename KVT, int NRB, int NS, int NW, int SHW, int D>
const char* launch_t4(const DecodeParams& p, int* ws_prefix, bool skip_combine, hipStream_t s) {
  const int n_rg = ring_row_groups(p.rows, NRB, SHW);
  const int64_t waves = (int64_t)p.n_parts * p.heads_kv * n_rg;
  constexpr bool SH = SHW > 1;
  // shared-stage variant: 8 XCDs x (workgroups of a group) x ceil(groups / 8), a group being one (partition, kv head);
  // the workgroups of groups past the last exit at once
  const int grid = SH ? 8 * (n_rg / SHW) * ((p.n_parts * p.heads_kv + 7) / 8) : (int)((waves + NW - 1) / NW);
  const size_t lds = (size_t)(SH ? 1 : NW) * NS * Geom<KVT, D>::STAGE;
  auto kern = paged_decode_mfma_kernel<QT, KVT, NRB, NS, NW, SHW, D>;
  // the LDS opt-in is a per-device function attribute: set once per device, not on every launch
  static std::atomic<bool> lds_opted_in[64];  // (one flag array per instantiation; zero-initialised)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return "hipGetDevice failed";
  if (dev < 0 || dev >= 64 || !lds_opted_in[dev].load(std::memory_order_acquire)) {
    hipError_t e0 = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e0 != hipSuccess) return hipGetErrorString(e0);
    if (dev >= 0 && dev < 64) lds_opted_in[dev].store(true, std::memory_order_release);  // (setting it twice from two threads is harmless)
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, s, p, ws_prefix);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hipGetErrorString(e);
  if (skip_combine) return nullptr;
  // one wave per row as a rule, four when sequences span more than eight partitions on average; beyond 64 the wide
  // kernel (sixteen waves, 16-byte lanes, one round of loads), which costs more per row and pays only there
  // rows per workgroup: one per wave while the call has few rows (decode), more once that would mean tens of thousands
  // of workgroups (prefill chunks)
  const int rows_all = p.heads_kv * p.rows;
  const bool wide = (int64_t)p.n_parts > 64 * (int64_t)p.batch, four = !wide && (int64_t)p.n_parts > 8 * (int64_t)p.batch;
  int rows_per_wg = (wide || four) ? 1 : 4;
  if (!wide && !four && (int64_t)rows_all * p.batch > 4096 && rows_all % 16 == 0) rows_per_wg = 16;  // four rows per wave, loaded together
  while ((int64_t)rows_all * p.batch / rows_per_wg > 8192 && rows_per_wg < 64) rows_per_wg *= 2;
  const dim3 cgrid((rows_all + rows_per_wg - 1) / rows_per_wg, p.batch, D > 128 ? 2 : 1);
  if (wide)
    hipLaunchKernelGGL((paged_decode_mfma_combine_wide_kernel<QT, 16>), cgrid, dim3(1024), 0, s, p, ws_prefix, rows_per_wg);
  else if (four)
    hipLaunchKernelGGL((paged_decode_mfma_combine_kernel<QT, 4>), cgrid, dim3(256), 0, s, p, ws_prefix, rows_per_wg);
  else if (rows_per_wg >= 16)
    hipLaunchKernelGGL((paged_decode_mfma_combine_kernel<QT, 1, true>), cgrid, dim3(256), 0, s, p, ws_prefix, rows_per_wg);
  else
    hipLaunchKernelGGL((paged_decode_mfma_combine_kernel<QT, 1>), cgrid, dim3(256), 0, s, p, ws_prefix, rows_per_wg);
  e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}

// Row blocks (16 query rows each) per wave: one up to 16 rows per kv head, else two -- one always at head dim 256,
// where two blocks of accumulators and operands do not fit the register file.
int row_blocks_for(int rows, int dim) { return (rows <= 16 || dim == 256) ? 1 : 2; }

// Waves per LDS ring.  Up to 32 rows per kv head there is one row group and every wave has its own ring.  Beyond, the
// 32-row groups of a kv head would each fetch the same K/V tiles: 8, 4 or 2 of them share one ring (a fraction of the
// fetch instructions per wave, one trip through the memory system per tile); an odd count is rounded up by one idle
// row group.  Eight waves a compute unit either way (accumulators of two row blocks fit ordinary vector registers);
// the ring takes the LDS that leaves (a 16-bit stage is 16 KiB, an fp8 one 8.25 KiB).
// (128-byte rows, fp8 or head dim 64, have four fetch instructions per K tile, 64-byte rows two.  Head dim 256 has one
// row block per wave: unshared waves and rings of two or four keep their accumulators in AGPRs and run one wave per
// SIMD; a ring of eight reads its K and V^T operands from LDS in portions -- K in two halves of the head dim, V^T four
// 16-column blocks at a time inside the value step -- so that a wave fits 256 registers and two run per SIMD: 128
// query rows per trip of a K/V tile through the memory system instead of 64, half the fetch instructions per wave.)
int ring_waves_for(int rows, int nrb, int max_ring) {
  const int n = row_groups(rows, nrb);
  if (n <= 1) return 1;
  const int even = (n + 1) / 2 * 2;
  if (even % 8 == 0 && max_ring >= 8) return 8;
  if (even % 4 == 0 && max_ring >= 4) return 4;
  return 2;
}
// Largest ring for a row width: a ring splits the fetch instructions of a K tile (one per KiB: 8, 4 or 2 for rows of
// 256, 128 or 64 bytes; 16 for the 512-byte rows of a 16-bit cache at head dim 256) evenly over its waves.
int max_ring_for(int dim, bool fp8) {
  const int row = dim * (fp8 ? 1 : 2);
  return (row == 256 || row == 512) ? 8 : (row == 64 ? 2 : 4);
}

template <typename QT, typename KVT, int D>
const char* launch_t2(const DecodeParams& p, int* ws_prefix, bool skip_combine, hipStream_t s) {
  constexpr bool SMALL = Geom<KVT, D>::ROW <= 128;  // 8 KiB stages or less: eight unshared waves a CU, four-deep pair rings
  constexpr bool WIDE = Geom<KVT, D>::ROW == 512;   // 32 KiB stages: two unshared waves per workgroup
  constexpr int NWU = SMALL ? 8 : (WIDE ? 2 : 4);   // unshared waves per workgroup (two stages each fill the LDS)
  if (p.rows <= 16) return launch_t4<QT, KVT, 1, 2, NWU, 1, D>(p, ws_prefix, skip_combine, s);
  constexpr int NRB = D == 256 ? 1 : 2;  // == row_blocks_for(rows > 16, D)
  switch (ring_waves_for(p.rows, NRB, max_ring_for(D, Geom<KVT, D>::FP8))) {
    case 1: return launch_t4<QT, KVT, NRB, 2, NWU, 1, D>(p, ws_prefix, skip_combine, s);
    // Stages per ring: as many as the LDS of a compute unit holds for its eight waves, up to eight -- half a ring is read
    // per barrier while the other half is refilled, so eight stages mean one barrier per four tiles (8 x 512-token
    // chunks on 4 K prefixes: 424 us with four stages, 406 with eight).
    case 2: return launch_t4<QT, KVT, NRB, SMALL ? (Geom<KVT, D>::ROW == 64 ? 8 : 4) : 2, 2, 2, D>(p, ws_prefix, skip_combine, s);
    case 4:
      if constexpr (Geom<KVT, D>::NI >= 4) return launch_t4<QT, KVT, NRB, SMALL ? 8 : 4, 4, 4, D>(p, ws_prefix, skip_combine, s);
      return "MFMA kernel: no ring of four waves for this row width";
    default:
      if constexpr (!SMALL) return launch_t4<QT, KVT, NRB, Geom<KVT, D>::STAGE <= 16384 ? 8 : 4, 8, 8, D>(p, ws_prefix, skip_combine, s);
      return "MFMA kernel: no ring of eight waves for this row width";
  }
}

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

}  // namespace

bool mfma_supported(int q_len, int heads, int heads_kv, int dim, int page_size, int q_dtype, int kv_dtype, float softcap) {
  (void)q_len; (void)heads; (void)heads_kv; (void)softcap;
  const bool fp8 = kv_dtype == MI355_DT_FP8_E4M3FN;
  if (!(dim == 64 || dim == 128 || dim == 256)) return false;
  if (!(page_size == 16 || page_size % kCT == 0)) return false;
  if (!fp8 && kv_dtype != q_dtype) return false;
  return true;
}

// Number of equal ranges the tile stream is cut into: one wave per (range, kv head, row group), sized so
// that every compute unit holds one (16-bit KV) or two (fp8 KV, half the LDS per stage) workgroups.
int mfma_num_parts(int heads_kv, int rows, int dim, int kv_dtype, int compute_units) {
  const bool fp8 = kv_dtype == MI355_DT_FP8_E4M3FN;
  const int nrb = row_blocks_for(rows, dim), shw = ring_waves_for(rows, nrb, max_ring_for(dim, fp8));
  const int n_rg = ring_row_groups(rows, nrb, shw);
  // resident waves per CU: eight with 128-byte rows (fp8, or head dim 64; LDS-limited) and for shared rings (accumulators in ordinary
  // vector registers, two waves per SIMD), four for unshared 16-bit waves (LDS-limited: 2 x 16 KiB stages each)
  const int waves_per_cu = dim == 256 ? (shw == 8 ? 8 : (shw > 1 || fp8) ? 4 : 2) : ((fp8 || dim == 64 || shw > 1) ? 8 : 4);
  const int64_t waves = (int64_t)compute_units * waves_per_cu;
  int64_t parts = waves / ((int64_t)heads_kv * n_rg);
  return parts < 1 ? 1 : (int)parts;
}

// [part_o: 2*n_parts slots x heads_kv*rows x dim fp32][part_lse: 2*n_parts x heads_kv*rows fp32][records: (batch+1) x int4]
size_t mfma_workspace_bytes(int n_parts, int heads_kv, int rows, int dim, int batch) {
  size_t slots = (size_t)2 * n_parts * heads_kv * rows;
  return align256(slots * dim * sizeof(float)) + align256(slots * sizeof(float)) + align256((size_t)(batch + 1) * 4 * sizeof(int));
}

const char* launch_mfma(const DecodeParams& p_in, int q_dtype, int kv_dtype, bool skip_combine, hipStream_t s) {
  DecodeParams p = p_in;
  // The kernel applies the score scale after taking row maxima, which needs it positive: move the sign into the
  // query, and replace a zero scale (uniform attention) by a tiny positive one so masked -inf scores stay -inf.
  float& signed_scale = p.softcap > 0.f ? p.inv_cap_scale : p.score_scale;
  p.negate_q = signed_scale < 0.f ? 1 : 0;
  signed_scale = fabsf(signed_scale);
  if (!(p.softcap > 0.f) && signed_scale < 1e-30f) signed_scale = 1e-30f;
  // Calls with many query rows (multi-token decode, prefill chunks) keep their partial rows in the query's 16-bit type, as the
  // reference does for every call (its Output_partial has the op's dtype, gqa_decode_paged.py:216-217,718-722): half the
  // bytes written by the attention kernel and read by the merge.  The log-sum-exps stay fp32, and so do the rows of
  // single-token decode.  (The sixteen-wave merge of very long single sequences reads fp32 rows only.)
  {
    const int64_t rows_all = (int64_t)p.heads_kv * p.rows;
    const bool wide = (int64_t)p.n_parts > 64 * (int64_t)p.batch;
    p.part16 = (!wide && p.rows > p.group && rows_all * p.batch > 4096) ? 1 : 0;  // (rows == group: one query token)
  }
  size_t slots = (size_t)2 * p.n_parts * p.heads_kv * p.rows;
  char* ws = (char*)p_in.part_o;
  p.part_o = (float*)ws;
  p.part_lse = (float*)(ws + align256(slots * p.dim * sizeof(float)));
  int* ws_prefix = (int*)(ws + align256(slots * p.dim * sizeof(float)) + align256(slots * sizeof(float)));
  // the kernel addresses pool rows with 32 bits
  const int64_t pool_rows = p.kv_starts ? INT32_MAX - 1 : (p.contig_stride ? (int64_t)p.batch * p.contig_stride : p.n_pages * p.page_size);
  if (pool_rows >= INT32_MAX) return "MFMA kernel: the KV pool has 2^31 or more rows";
  if (p.dim == 64) {
    if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_BF16) return launch_t2<bf16_tag, bf16_tag, 64>(p, ws_prefix, skip_combine, s);
    if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP16) return launch_t2<fp16_tag, fp16_tag, 64>(p, ws_prefix, skip_combine, s);
    if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_t2<bf16_tag, fp8_tag, 64>(p, ws_prefix, skip_combine, s);
    if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_t2<fp16_tag, fp8_tag, 64>(p, ws_prefix, skip_combine, s);
    return "MFMA kernel: unsupported (q_dtype, kv_dtype) pair";
  }
  if (p.dim == 256) {
    if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_BF16) return launch_t2<bf16_tag, bf16_tag, 256>(p, ws_prefix, skip_combine, s);
    if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP16) return launch_t2<fp16_tag, fp16_tag, 256>(p, ws_prefix, skip_combine, s);
    if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_t2<bf16_tag, fp8_tag, 256>(p, ws_prefix, skip_combine, s);
    if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_t2<fp16_tag, fp8_tag, 256>(p, ws_prefix, skip_combine, s);
    return "MFMA kernel: unsupported (q_dtype, kv_dtype) pair";
  }
  if (p.dim != 128) return "MFMA kernel: unsupported head dim";
  if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_BF16) return launch_t2<bf16_tag, bf16_tag, 128>(p, ws_prefix, skip_combine, s);
  if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP16) return launch_t2<fp16_tag, fp16_tag, 128>(p, ws_prefix, skip_combine, s);
  if (q_dtype == MI355_DT_BF16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_t2<bf16_tag, fp8_tag, 128>(p, ws_prefix, skip_combine, s);
  if (q_dtype == MI355_DT_FP16 && kv_dtype == MI355_DT_FP8_E4M3FN) return launch_t2<fp16_tag, fp8_tag, 128>(p, ws_prefix, skip_combine, s);
  return "MFMA kernel: unsupported (q_dtype, kv_dtype) pair";
}

}  // namespace mi355
