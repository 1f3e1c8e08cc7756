// Dense matrix-instruction rate probe for MI355X (gfx950).  Stand-alone HIP program:
//   hipcc --offload-arch=gfx950 -O3 tileops_amd/perf/mfma_rate_probe.hip -o mfma_rate_probe && ./mfma_rate_probe
// It plays the role of the reference's GEMM-throughput calibrator (benchmarks/hardware/compute/gemm_throughput.py, whose
// figure is the tensor_core calibration of src/tileops/perf/profiles/h200.yaml:15-21): what fraction of the published
// dense rate the matrix pipes sustain when nothing else limits them.  Operands stay in registers, every wave keeps
// several independent accumulator chains going, all compute units are filled; the only limits left are the issue rate
// of the instruction and the power the part allows itself under a saturating matrix load.  The figures it prints are
// what tileops_amd/perf/profiles/mi355x.yaml records as matrix.*.calibration, and the ceiling against which the
// attention kernels' matrix rates (eight query tokens, prefill chunks) are to be read.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <vector>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

constexpr int kChains = 8;      // independent accumulators per wave: dependent instructions are kChains apart
constexpr int kIters = 4096;    // loop trips; kChains matrix instructions each

// KIND 0: v_mfma_f32_16x16x32_bf16   1: v_mfma_f32_16x16x32_f16   2: v_mfma_f32_32x32x16_bf16
//      3: v_mfma_f32_16x16x128_f8f6f4 (fp8 x fp8)                 4: v_mfma_f32_32x32x64_f8f6f4 (fp8 x fp8)
// The instructions are written as inline assembly with the accumulator tied in place: through the builtins the compiler
// shuffles the loop-carried accumulators between register files on every trip, and the probe would time its moves.
template <int KIND> struct Op;
template <> struct Op<0> {
  using Acc = f32x4;
  static constexpr double flop = 2.0 * 16 * 16 * 32;
  static __device__ __forceinline__ void run(u32x4 a, u32x4 b, i32x8, i32x8, Acc& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
};
template <> struct Op<1> {
  using Acc = f32x4;
  static constexpr double flop = 2.0 * 16 * 16 * 32;
  static __device__ __forceinline__ void run(u32x4 a, u32x4 b, i32x8, i32x8, Acc& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
};
template <> struct Op<2> {
  using Acc = f32x16;
  static constexpr double flop = 2.0 * 32 * 32 * 16;
  static __device__ __forceinline__ void run(u32x4 a, u32x4 b, i32x8, i32x8, Acc& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
};
template <> struct Op<3> {
  using Acc = f32x4;
  static constexpr double flop = 2.0 * 16 * 16 * 128;
  static __device__ __forceinline__ void run(u32x4, u32x4, i32x8 a, i32x8 b, Acc& c) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
};
template <> struct Op<4> {
  using Acc = f32x16;
  static constexpr double flop = 2.0 * 32 * 32 * 64;
  static __device__ __forceinline__ void run(u32x4, u32x4, i32x8 a, i32x8 b, Acc& c) {
    asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
};

template <int KIND>
__global__ __launch_bounds__(256) void k_mfma(const u32x4* __restrict__ seed, float* __restrict__ sink, int iters) {
  using O = Op<KIND>;
  // operands come from memory once, so the compiler cannot fold the products; small finite values in every format
  const u32x4 a = seed[threadIdx.x & 63], b = seed[64 + (threadIdx.x & 63)];
  const u32x4 a2 = seed[128 + (threadIdx.x & 63)], b2 = seed[192 + (threadIdx.x & 63)];
  const i32x8 a8 = {(int)a[0], (int)a[1], (int)a[2], (int)a[3], (int)a2[0], (int)a2[1], (int)a2[2], (int)a2[3]};
  const i32x8 b8 = {(int)b[0], (int)b[1], (int)b[2], (int)b[3], (int)b2[0], (int)b2[1], (int)b2[2], (int)b2[3]};
  typename O::Acc acc[kChains];
#pragma unroll
  for (int c = 0; c < kChains; c++)
#pragma unroll
    for (int e = 0; e < (int)(sizeof(typename O::Acc) / 4); e++) acc[c][e] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int c = 0; c < kChains; c++) O::run(a, b, a8, b8, acc[c]);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < kChains; c++)
#pragma unroll
    for (int e = 0; e < (int)(sizeof(typename O::Acc) / 4); e++) s += acc[c][e];
  if (s == 12345.678f) sink[blockIdx.x] = s;  // (never true; keeps the chains alive)
}

template <int KIND>
double measure(const u32x4* seed, float* sink, int cus, int wg_per_cu, const char* name, double peak_tflops) {
  const int grid = cus * wg_per_cu;  // 4 waves per workgroup = one per SIMD; wg_per_cu of them share a compute unit
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int w = 0; w < 2; w++) hipLaunchKernelGGL(k_mfma<KIND>, dim3(grid), dim3(256), 0, 0, seed, sink, kIters);
  CK(hipDeviceSynchronize());
  std::vector<float> ms;
  for (int r = 0; r < 7; r++) {
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(k_mfma<KIND>, dim3(grid), dim3(256), 0, 0, seed, sink, kIters);
    CK(hipEventRecord(e1, 0));
    CK(hipEventSynchronize(e1));
    float t;
    CK(hipEventElapsedTime(&t, e0, e1));
    ms.push_back(t);
  }
  std::sort(ms.begin(), ms.end());
  const double t = ms[ms.size() / 2] * 1e-3;
  const double flop = (double)grid * 4 * kIters * kChains * Op<KIND>::flop;
  const double tf = flop / t / 1e12;
  printf("| %-34s | %d | %8.1f | %7.1f | %6.1f | %5.3f |\n", name, wg_per_cu * 4, ms[ms.size() / 2] * 1e3, tf, peak_tflops, tf / peak_tflops);
  return tf;
}

int main() {
  int dev = 0, cus = 0;
  CK(hipGetDevice(&dev));
  CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  std::vector<uint32_t> host(256 * 4);
  // bf16 1.0 pairs (0x3f803f80) are also small finite fp16 (1.875) and fp8-e4m3fn (0x3f = 1.875, 0x80 = -0) values
  for (auto& w : host) w = 0x3f803f80u;
  u32x4* seed;
  float* sink;
  CK(hipMalloc(&seed, host.size() * 4));
  CK(hipMalloc(&sink, (size_t)cus * 8 * sizeof(float)));
  CK(hipMemcpy(seed, host.data(), host.size() * 4, hipMemcpyHostToDevice));
  printf("compute units: %d; %d accumulator chains per wave, %d trips\n", cus, kChains, kIters);
  printf("| instruction | waves/CU | us | TFLOP/s | published dense peak | fraction |\n|---|---:|---:|---:|---:|---:|\n");
  for (int wg : {1, 2}) {
    measure<0>(seed, sink, cus, wg, "v_mfma_f32_16x16x32_bf16", 2500.0);
    measure<1>(seed, sink, cus, wg, "v_mfma_f32_16x16x32_f16", 2500.0);
    measure<2>(seed, sink, cus, wg, "v_mfma_f32_32x32x16_bf16", 2500.0);
    measure<3>(seed, sink, cus, wg, "v_mfma_f32_16x16x128_f8f6f4 (fp8)", 5000.0);
    measure<4>(seed, sink, cus, wg, "v_mfma_f32_32x32x64_f8f6f4 (fp8)", 5000.0);
  }
  CK(hipFree(seed));
  CK(hipFree(sink));
  return 0;
}
