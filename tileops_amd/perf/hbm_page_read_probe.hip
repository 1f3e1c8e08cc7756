// HBM read-bandwidth probe for paged KV access patterns on MI355X (gfx950).  Stand-alone HIP program:
//   hipcc --offload-arch=gfx950 -O3 tileops_amd/perf/hbm_page_read_probe.hip -o hbm_page_read_probe && ./hbm_page_read_probe
// It plays the role of the reference's STREAM-style calibrator (benchmarks/hardware/memory/hbm_saturation.cu):
// the figures it prints are what tileops_amd/perf/profiles/mi355x.yaml records and what the decode kernel's
// load strategy (non-temporal direct-to-LDS loads of whole K/V rows) was chosen from.
//
// Pool: 1 Mi tokens x 2 KiB (8 kv heads x 128 x bf16) = 2 GiB, read in 128 KiB pages (64 tokens) taken from a
// random permutation; every pattern reads 1 GiB per launch.
//   stream      : linear 128-bit loads, default or non-temporal
//   head-slice  : wave = kv head, each wave instruction reads four 256-byte rows (one per 16 lanes) into registers
//   mfma-operand: wave = kv head, lane (l%16 = token, l/16 = 64-byte quarter of the row): the layout an MFMA A
//                 operand wants, read straight from global memory
//   page-linear : the workgroup reads the 128 KiB page front to back
//   lds-direct  : head-slice addresses, global_load_lds_dwordx4 into a per-wave LDS ring of NB x 8 KiB
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <numeric>
#include <random>
#include <vector>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
#define LDSP(T, p) ((__attribute__((address_space(3))) T*)(p))

template <int NT> __device__ __forceinline__ u32x4 ld(const u32x4* p) { return NT ? __builtin_nontemporal_load(p) : *p; }

template <int U, int NT>
__global__ __launch_bounds__(256) void k_stream(const u32x4* __restrict__ src, size_t n_vec, unsigned* sink) {
  u32x4 acc = {0, 0, 0, 0};
  const size_t chunk = (size_t)256 * U;
  for (size_t c = blockIdx.x; c < n_vec / chunk; c += gridDim.x) {
    const u32x4* p = src + c * chunk + threadIdx.x;
    u32x4 v[U];
#pragma unroll
    for (int i = 0; i < U; i++) v[i] = ld<NT>(p + (size_t)i * 256);
#pragma unroll
    for (int i = 0; i < U; i++) acc ^= v[i];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1;
}

// MODE 0 head-slice, 1 mfma-operand, 2 page-linear; 8 waves per workgroup
template <int MODE, int NT>
__global__ __launch_bounds__(512) void k_page(const char* __restrict__ pool, const int* __restrict__ pages, int n_pages, unsigned* sink) {
  u32x4 acc = {0, 0, 0, 0};
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63;
  for (int it = blockIdx.x; it < n_pages; it += gridDim.x) {
    const char* base = pool + (size_t)pages[it] * (64 * 2048);
    u32x4 v[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
      if (MODE == 0) v[i] = ld<NT>((const u32x4*)(base + (4 * i + (l >> 4)) * 2048 + wave * 256 + (l & 15) * 16));
      else if (MODE == 1) v[i] = ld<NT>((const u32x4*)(base + (16 * (i >> 2) + (l & 15)) * 2048 + wave * 256 + (4 * (i & 3) + (l >> 4)) * 16));
      else v[i] = ld<NT>((const u32x4*)(base + ((size_t)i * 512 + threadIdx.x) * 16));
    }
#pragma unroll
    for (int i = 0; i < 16; i++) acc ^= v[i];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1;
}

template <int NT> __device__ __forceinline__ void dma16(unsigned lds_addr, unsigned voff, const char* sbase) {
  unsigned long long v = (unsigned long long)sbase;
  unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  sbase = (const char*)(((unsigned long long)hi << 32) | lo);
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  if (NT) asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  else asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// NW waves per workgroup, 8/NW workgroups share a page; ring of NB half-page (32-token, 8 KiB) buffers per wave
template <int NW, int NB, int NT>
__global__ __launch_bounds__(NW * 64) void k_lds(const char* __restrict__ pool, const int* __restrict__ pages, int n_pages, unsigned* sink) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), l = threadIdx.x & 63;
  constexpr int WPP = 8 / NW;
  const int head = (blockIdx.x % WPP) * NW + wave, grp = blockIdx.x / WPP, ngrp = gridDim.x / WPP;
  const unsigned my = __builtin_amdgcn_readfirstlane((unsigned)(size_t)LDSP(char, lds)) + wave * (NB * 8192);
  int n_half = 0;
  for (int it = grp; it < n_pages; it += ngrp) n_half += 2;
  const unsigned voff = (l >> 4) * 2048 + (l & 15) * 16;
  auto issue = [&](int h) {
    const int pg = __builtin_amdgcn_readfirstlane(pages[grp + (h >> 1) * ngrp]);
    const char* base = pool + (size_t)pg * (64 * 2048) + (h & 1) * (32 * 2048) + head * 256;
#pragma unroll
    for (int i = 0; i < 8; i++) dma16<NT>(my + (h % NB) * 8192 + i * 1024, voff, base + i * 4 * 2048);
  };
  for (int h = 0; h < NB - 1 && h < n_half; h++) issue(h);
  unsigned acc = 0;
  for (int h = 0; h < n_half; h++) {
    if (h + NB - 1 < n_half) { issue(h + NB - 1); wait_vm<(NB - 1) * 8>(); } else wait_vm<0>();
    acc ^= *LDSP(volatile unsigned, lds + wave * (NB * 8192) + (h % NB) * 8192 + l * 4);
  }
  if (acc == 0x12345678u) sink[0] = 1;
}

static float time_median(const std::function<void()>& f, int reps = 9) {
  hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  f(); CK(hipDeviceSynchronize());
  std::vector<float> t;
  for (int r = 0; r < reps; r++) { CK(hipEventRecord(a)); f(); CK(hipEventRecord(b)); CK(hipEventSynchronize(b)); float ms; CK(hipEventElapsedTime(&ms, a, b)); t.push_back(ms); }
  std::sort(t.begin(), t.end());
  return t[t.size() / 2];
}

int main() {
  hipDeviceProp_t prop; CK(hipGetDeviceProperties(&prop, 0));
  printf("device %s %s CUs %d\n", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  const size_t n_tok = 1 << 20, bytes = n_tok * 2048;
  char* pool; CK(hipMalloc(&pool, bytes)); CK(hipMemset(pool, 1, bytes));
  unsigned* sink; CK(hipMalloc(&sink, 4));
  const int n_pages = n_tok / 64, np = n_pages / 2;
  std::vector<int> hp(n_pages); std::iota(hp.begin(), hp.end(), 0);
  std::mt19937 rng(1); std::shuffle(hp.begin(), hp.end(), rng);
  int* pages; CK(hipMalloc(&pages, n_pages * 4)); CK(hipMemcpy(pages, hp.data(), n_pages * 4, hipMemcpyHostToDevice));
  const double gb = (double)np * 64 * 2048 / 1e9;
  auto rep = [&](const char* name, int grid, float ms) { printf("%-40s grid %5d  %8.1f us  %7.1f GB/s  %5.1f %% of 8 TB/s\n", name, grid, ms * 1e3, gb / (ms * 1e-3), gb / (ms * 1e-3) / 80.0); fflush(stdout); };
  const size_t nvec = (size_t)np * 64 * 2048 / 16;
  for (int grid : {512, 2048}) {
    rep("stream, default loads", grid, time_median([&] { k_stream<4, 0><<<grid, 256>>>((const u32x4*)pool, nvec, sink); }));
    rep("stream, non-temporal loads", grid, time_median([&] { k_stream<4, 1><<<grid, 256>>>((const u32x4*)pool, nvec, sink); }));
  }
  for (int grid : {256, 1024}) {
    rep("head-slice -> registers, default", grid, time_median([&] { k_page<0, 0><<<grid, 512>>>(pool, pages, np, sink); }));
    rep("head-slice -> registers, non-temporal", grid, time_median([&] { k_page<0, 1><<<grid, 512>>>(pool, pages, np, sink); }));
    rep("mfma-operand -> registers, default", grid, time_median([&] { k_page<1, 0><<<grid, 512>>>(pool, pages, np, sink); }));
    rep("mfma-operand -> registers, non-temporal", grid, time_median([&] { k_page<1, 1><<<grid, 512>>>(pool, pages, np, sink); }));
    rep("page-linear -> registers, default", grid, time_median([&] { k_page<2, 0><<<grid, 512>>>(pool, pages, np, sink); }));
    rep("page-linear -> registers, non-temporal", grid, time_median([&] { k_page<2, 1><<<grid, 512>>>(pool, pages, np, sink); }));
  }
#define RUN_LDS(NW, NB, NT, G) { CK(hipFuncSetAttribute((const void*)k_lds<NW, NB, NT>, hipFuncAttributeMaxDynamicSharedMemorySize, NW * NB * 8192)); \
    char nm[80]; snprintf(nm, 80, "lds-direct %d waves x %d bufs, %s", NW, NB, NT ? "non-temporal" : "default"); \
    rep(nm, G, time_median([&] { k_lds<NW, NB, NT><<<G, NW * 64, NW * NB * 8192>>>(pool, pages, np, sink); })); }
  RUN_LDS(4, 2, 0, 256); RUN_LDS(4, 2, 1, 256); RUN_LDS(4, 4, 1, 256); RUN_LDS(8, 2, 1, 256); RUN_LDS(4, 2, 1, 1024);
  CK(hipDeviceSynchronize());
  return 0;
}
