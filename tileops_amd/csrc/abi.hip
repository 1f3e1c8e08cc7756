// extern "C" entry points of libmi355_tileops: argument validation, kernel choice, launch.
// Never throws, never aborts, never synchronises, never allocates device memory.
#include <limits.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>

#include "common.h"

using namespace mi355;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Architecture of the current device, asked once per device: 1 = gfx950, -1 = something else, 0 = not asked yet.
// The kernels are gfx950 code objects (direct-to-LDS loads, transpose reads, the 128-deep fp8 matrix instruction);
// the reference refuses by architecture before building a kernel (src/tileops/kernels/kernel_base.py:98-112).
constexpr int kMaxDevices = 64;
std::atomic<int> g_arch_ok[kMaxDevices];
std::atomic<int> g_cu_count[kMaxDevices];

int check_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) {
    (void)hipGetLastError();
    return fail(MI355_EDEVICE, "no HIP device is current (these kernels need a gfx950 GPU)");
  }
  int known = dev < kMaxDevices ? g_arch_ok[dev].load(std::memory_order_relaxed) : 0;
  if (known == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
      (void)hipGetLastError();
      return fail(MI355_EDEVICE, "cannot read the properties of HIP device %d", dev);
    }
    known = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
    if (dev < kMaxDevices) g_arch_ok[dev].store(known, std::memory_order_relaxed);
    if (known < 0) return fail(MI355_EDEVICE, "HIP device %d is %s; this library holds gfx950 (MI355X) code only", dev, prop.gcnArchName);
  }
  if (known < 0) return fail(MI355_EDEVICE, "HIP device %d is not a gfx950 (MI355X) GPU", dev);
  return MI355_OK;
}

bool is_q_dtype(int d) { return d == MI355_DT_BF16 || d == MI355_DT_FP16; }
bool is_kv_dtype(int d) { return d == MI355_DT_BF16 || d == MI355_DT_FP16 || d == MI355_DT_FP8_E4M3FN; }

// Shape-only checks shared by the workspace query and the launch.
int check_shape(int batch, int q_len, int heads, int heads_kv, int dim, int page_size, int q_dtype, int kv_dtype) {
  if (batch < 0) return fail(MI355_EINVAL, "batch must be non-negative, got %d", batch);
  if (q_len <= 0) return fail(MI355_EINVAL, "q_len must be positive, got %d", q_len);
  if (heads <= 0) return fail(MI355_EINVAL, "heads must be positive, got %d", heads);
  if (heads_kv <= 0) return fail(MI355_EINVAL, "heads_kv must be positive, got %d", heads_kv);
  if (heads % heads_kv != 0) return fail(MI355_EINVAL, "heads must be divisible by heads_kv (%d %% %d)", heads, heads_kv);
  if (dim <= 0) return fail(MI355_EINVAL, "dim must be positive, got %d", dim);
  if (page_size <= 0) return fail(MI355_EINVAL, "page_size must be positive, got %d", page_size);
  if (!is_q_dtype(q_dtype)) return fail(MI355_EINVAL, "q_dtype must be bf16 or fp16, got code %d", q_dtype);
  if (!is_kv_dtype(kv_dtype)) return fail(MI355_EINVAL, "kv_dtype must be bf16, fp16 or fp8_e4m3fn, got code %d", kv_dtype);
  if (kv_dtype != MI355_DT_FP8_E4M3FN && kv_dtype != q_dtype)
    return fail(MI355_EINVAL, "a 16-bit kv_dtype must equal q_dtype (q code %d, kv code %d)", q_dtype, kv_dtype);
  if (dim != 64 && dim != 128 && dim != 256)
    return fail(MI355_EUNSUPPORTED, "head dim %d is not served (64, 128 or 256)", dim);
  if (batch > 65535) return fail(MI355_EUNSUPPORTED, "batch %d exceeds 65535", batch);
  return MI355_OK;
}

struct Plan {
  int kernel;        // MI355_KERNEL_GENERIC or MI355_KERNEL_MFMA
  int max_splits;    // generic
  int split_tokens;  // generic
  int n_parts;       // mfma
  size_t part_o_bytes, part_lse_bytes;
};

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

constexpr int kPlanCuCount = 256;    // MI355X: 8 XCDs x 32 compute units
constexpr int kMaxMfmaParts = 4096;  // the kernel's 32-bit partition arithmetic holds up to here

// for_launch: the call is about to run on the current device, whose compute-unit count sizes the MFMA kernel's partition
// count (never more than the 256 of an MI355X, which is what a workspace query plans for without touching any device, so a
// workspace sized by the query always holds the launch's plan).
int make_plan(int batch, int q_len, int heads, int heads_kv, int dim, int page_size, int64_t max_blocks_per_seq, int q_dtype,
              int kv_dtype, float softcap, int num_split_in, int kernel, Plan* plan, bool for_launch = false) {
  if (max_blocks_per_seq < 0) return fail(MI355_EINVAL, "max_blocks_per_seq must be non-negative");
  if (num_split_in < 0) return fail(MI355_EINVAL, "num_split must be non-negative, got %d", num_split_in);
  const int rows = q_len * (heads / heads_kv);
  bool mfma_ok = mfma_supported(q_len, heads, heads_kv, dim, page_size, q_dtype, kv_dtype, softcap);
  if (kernel == MI355_KERNEL_MFMA && !mfma_ok)
    return fail(MI355_EUNSUPPORTED, "the MFMA kernel does not serve this shape (dim %d, page_size %d, rows %d, dtypes %d/%d)",
                dim, page_size, rows, q_dtype, kv_dtype);
  if (kernel != MI355_KERNEL_AUTO && kernel != MI355_KERNEL_GENERIC && kernel != MI355_KERNEL_MFMA)
    return fail(MI355_EINVAL, "unknown kernel selector %d", kernel);
  plan->kernel = (kernel == MI355_KERNEL_GENERIC || !mfma_ok) ? MI355_KERNEL_GENERIC : MI355_KERNEL_MFMA;
  if (plan->kernel == MI355_KERNEL_GENERIC) {
    // Fixed-length splits of ~512 tokens, at most 64 per sequence, bounded by what the table can address.
    plan->split_tokens = 512;
    int64_t max_ctx = max_blocks_per_seq * (int64_t)page_size;
    int64_t cap = (max_ctx + plan->split_tokens - 1) / plan->split_tokens;
    if (cap < 1) cap = 1;
    int ms = num_split_in > 0 ? num_split_in : 64;
    if (ms > 1024) ms = 1024;
    if (ms > cap) ms = (int)cap;
    plan->max_splits = ms;
    plan->n_parts = 0;
    size_t slots = (size_t)batch * ms;
    plan->part_o_bytes = ms > 1 ? align256(slots * heads_kv * rows * dim * sizeof(float)) : 0;
    plan->part_lse_bytes = ms > 1 ? align256(slots * heads_kv * rows * sizeof(float)) : 0;
  } else {
    plan->max_splits = 0;
    plan->split_tokens = 0;
    // num_split > 0 fixes the partition count (what the kernel class's autotuner varies); 0 = one range per resident wave
    const int cus = for_launch ? (device_cu_count() < kPlanCuCount ? device_cu_count() : kPlanCuCount) : kPlanCuCount;
    plan->n_parts = num_split_in > 0 ? (num_split_in < kMaxMfmaParts ? num_split_in : kMaxMfmaParts) : mfma_num_parts(heads_kv, rows, dim, kv_dtype, cus);
    size_t total = mfma_workspace_bytes(plan->n_parts, heads_kv, rows, dim, batch);
    plan->part_o_bytes = total;  // the MFMA launcher lays out its own workspace
    plan->part_lse_bytes = 0;
  }
  return MI355_OK;
}

// What a prefill chunk adds to a decode call (all zero for the decode entry points).
struct Extras {
  const int32_t* cu_q = nullptr;
  int len_excludes_new = 0;
  const int32_t* kv_starts = nullptr;
  int scale_per_tensor = 0;
  float* final_o = nullptr;
  float* final_lse = nullptr;
  const float* init_o = nullptr;
  const float* init_lse = nullptr;
};

// One decode call, paged (block_table/seqlens given) or contiguous (contig_stride > 0, uniform_len).
int run_decode(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
               const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride, int64_t contig_stride,
               int uniform_len, void* out, void* workspace, size_t workspace_bytes, int batch, int q_len, int heads,
               int heads_kv, int dim, int page_size, int64_t n_phys_tokens, int q_dtype, int kv_dtype, float sm_scale,
               float softcap, int causal, int num_split, int kernel, void* hip_stream, const Extras& ex = Extras()) {
  const bool skip_combine = (kernel & kKernelFlagSkipCombine) != 0;
  kernel &= ~kKernelFlagSkipCombine;
  const bool fp8 = kv_dtype == MI355_DT_FP8_E4M3FN;
  if (fp8 && (!k_scale || !v_scale)) return fail(MI355_EINVAL, "k_scale and v_scale are required with an fp8 KV cache");
  if (!fp8 && (k_scale || v_scale)) return fail(MI355_EINVAL, "k_scale and v_scale must be null unless kv_dtype is fp8_e4m3fn");
  if (!(softcap >= 0.f)) return fail(MI355_EINVAL, "softcap must be non-negative");
  if (!(sm_scale == sm_scale)) return fail(MI355_EINVAL, "sm_scale is NaN");
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15)
    return fail(MI355_EINVAL, "q, k, v and out must be 16-byte aligned");
  Plan plan;
  int rc = make_plan(batch, q_len, heads, heads_kv, dim, page_size, bt_row_stride, q_dtype, kv_dtype, softcap, num_split, kernel, &plan, true);
  if (rc) return rc;
  const size_t need = plan.part_o_bytes + plan.part_lse_bytes;
  if (need > 0) {
    if (!workspace) return fail(MI355_EWORKSPACE, "workspace of %zu bytes required, got null", need);
    if (workspace_bytes < need) return fail(MI355_EWORKSPACE, "workspace of %zu bytes required, got %zu", need, workspace_bytes);
    if ((uintptr_t)workspace & 255) return fail(MI355_EWORKSPACE, "workspace must be 256-byte aligned");
  }

  rc = check_device();
  if (rc) return rc;

  DecodeParams p;
  memset(&p, 0, sizeof(p));
  p.q = q;
  p.k = k;
  p.v = v;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.seqlens = seqlens;
  p.block_table = block_table;
  p.bt_row_stride = bt_row_stride;
  p.contig_stride = contig_stride;
  p.uniform_len = uniform_len;
  p.cu_q = ex.cu_q;
  p.len_excludes_new = ex.len_excludes_new;
  p.kv_starts = ex.kv_starts;
  p.scale_per_tensor = ex.scale_per_tensor;
  p.final_o = ex.final_o;
  p.final_lse = ex.final_lse;
  p.init_o = ex.init_o;
  p.init_lse = ex.init_lse;
  p.out = out;
  p.part_o = (float*)workspace;
  p.part_lse = (float*)((char*)workspace + plan.part_o_bytes);
  p.batch = batch;
  p.q_len = q_len;
  p.heads = heads;
  p.heads_kv = heads_kv;
  p.dim = dim;
  p.page_size = page_size;
  p.group = heads / heads_kv;
  p.rows = q_len * p.group;
  p.n_pages = n_phys_tokens / page_size;
  {
    // what one block-table row (contiguous cache: one sequence's share, passed as bt_row_stride tiles) can address
    const int64_t cap = bt_row_stride * (int64_t)page_size;
    p.max_len = cap > INT_MAX ? INT_MAX : (int)cap;
  }
  p.softcap = softcap;
  if (softcap > 0.f) {
    p.score_scale = sm_scale;
    p.cap_log2e = softcap * kLog2e;
    p.inv_cap_scale = sm_scale / softcap;
  } else {
    p.score_scale = sm_scale * kLog2e;
  }
  p.causal = causal ? 1 : 0;
  p.max_splits = plan.max_splits;
  p.split_tokens = plan.split_tokens;
  p.n_parts = plan.n_parts;

  hipStream_t s = (hipStream_t)hip_stream;
  const char* err;
  if (plan.kernel == MI355_KERNEL_GENERIC) {
    err = launch_generic(p, q_dtype, kv_dtype, s);
    if (!err && !skip_combine) err = launch_generic_combine(p, q_dtype, s);
  } else {
    err = launch_mfma(p, q_dtype, kv_dtype, skip_combine, s);
  }
  if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
  return MI355_OK;
}

// Scratch of the entry point that allocates nothing (mi355_gqa_paged_decode_static): one array per GPU, there from
// the moment the code object is loaded until the process ends.  Host code never uses the array's name as an address:
// the name is a host-side handle, the array's device address is asked for once per device and kept.
constexpr size_t kStaticScratchBytes = (size_t)80 << 20;  // every plan of the MFMA kernel fits (at most 67.6 MB)
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) {
    (void)hipGetLastError();
    return fail(MI355_EDEVICE, "no HIP device is current (these kernels need a gfx950 GPU)");
  }
  if (dev >= kMaxDevices) return fail(MI355_EUNSUPPORTED, "device index %d exceeds the %d devices the static scratch table holds", dev, kMaxDevices);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));  // this device's copy of the array (the current device's)
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return fail(MI355_ELAUNCH, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
    }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return MI355_OK;
}

}  // namespace

namespace mi355 {
int device_cu_count() {
  constexpr int kDefault = 256;  // MI355X: 8 XCDs x 32 compute units
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) {
    (void)hipGetLastError();
    return kDefault;
  }
  int n = dev < kMaxDevices ? g_cu_count[dev].load(std::memory_order_relaxed) : 0;
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return kDefault;
  }
  if (dev < kMaxDevices) g_cu_count[dev].store(n, std::memory_order_relaxed);
  return n;
}
}  // namespace mi355

extern "C" {

int mi355_abi_version(void) { return MI355_ABI_VERSION; }

const char* mi355_last_error(void) { return g_err; }

int mi355_gqa_paged_decode_workspace(int batch, int q_len, int heads, int heads_kv, int dim, int page_size,
                                     int64_t max_blocks_per_seq, int q_dtype, int kv_dtype, int num_split_in, int kernel,
                                     size_t* workspace_bytes, int* num_split_out, int* kernel_out) {
  int rc = check_shape(batch, q_len, heads, heads_kv, dim, page_size, q_dtype, kv_dtype);
  if (rc) return rc;
  Plan plan;
  // softcap does not change the plan; the MFMA kernel serves both settings
  rc = make_plan(batch, q_len, heads, heads_kv, dim, page_size, max_blocks_per_seq, q_dtype, kv_dtype, 0.f, num_split_in,
                 kernel & ~kKernelFlagSkipCombine, &plan);
  if (rc) return rc;
  if (workspace_bytes) *workspace_bytes = plan.part_o_bytes + plan.part_lse_bytes;
  if (num_split_out) *num_split_out = plan.kernel == MI355_KERNEL_GENERIC ? plan.max_splits : plan.n_parts;
  if (kernel_out) *kernel_out = plan.kernel;
  return MI355_OK;
}

int mi355_gqa_paged_decode(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                           const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride, void* out, void* workspace,
                           size_t workspace_bytes, int batch, int q_len, int heads, int heads_kv, int dim, int page_size,
                           int64_t n_phys_tokens, int q_dtype, int kv_dtype, float sm_scale, float softcap, int causal,
                           int num_split, int kernel, void* hip_stream) {
  int rc = check_shape(batch, q_len, heads, heads_kv, dim, page_size, q_dtype, kv_dtype);
  if (rc) return rc;
  if (batch == 0) return MI355_OK;
  if (!q || !k || !v || !seqlens || !block_table || !out)
    return fail(MI355_EINVAL, "q, k, v, seqlens, block_table and out must be non-null");
  if (n_phys_tokens <= 0 || n_phys_tokens % page_size != 0)
    return fail(MI355_EINVAL, "n_phys_tokens (%lld) must be a positive multiple of page_size (%d)", (long long)n_phys_tokens,
                page_size);
  if (bt_row_stride <= 0) return fail(MI355_EINVAL, "bt_row_stride must be positive");
  return run_decode(q, k, v, k_scale, v_scale, seqlens, block_table, bt_row_stride, 0, 0, out, workspace, workspace_bytes,
                    batch, q_len, heads, heads_kv, dim, page_size, n_phys_tokens, q_dtype, kv_dtype, sm_scale, softcap,
                    causal, num_split, kernel, hip_stream);
}

int mi355_gqa_paged_decode_static(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                  const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride, void* out, int batch,
                                  int q_len, int heads, int heads_kv, int dim, int page_size, int64_t n_phys_tokens, int q_dtype,
                                  int kv_dtype, float sm_scale, float softcap, int causal, int num_split, int kernel,
                                  void* hip_stream) {
  int rc = check_shape(batch, q_len, heads, heads_kv, dim, page_size, q_dtype, kv_dtype);
  if (rc) return rc;
  if (batch == 0) return MI355_OK;
  if (!q || !k || !v || !seqlens || !block_table || !out)
    return fail(MI355_EINVAL, "q, k, v, seqlens, block_table and out must be non-null");
  if (n_phys_tokens <= 0 || n_phys_tokens % page_size != 0)
    return fail(MI355_EINVAL, "n_phys_tokens (%lld) must be a positive multiple of page_size (%d)", (long long)n_phys_tokens,
                page_size);
  if (bt_row_stride <= 0) return fail(MI355_EINVAL, "bt_row_stride must be positive");
  if (kernel & kKernelFlagSkipCombine) return fail(MI355_EINVAL, "unknown kernel selector %d", kernel);
  Plan plan;
  rc = make_plan(batch, q_len, heads, heads_kv, dim, page_size, bt_row_stride, q_dtype, kv_dtype, softcap, num_split, kernel, &plan);
  if (rc) return rc;
  const size_t need = plan.part_o_bytes + plan.part_lse_bytes;
  if (need > kStaticScratchBytes)
    return fail(MI355_EWORKSPACE, "this call needs %zu bytes of scratch, the static buffer of mi355_gqa_paged_decode_static holds %zu: "
                "use mi355_gqa_paged_decode with a workspace of the caller's", need, kStaticScratchBytes);
  rc = check_device();
  if (rc) return rc;
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc) return rc;
  // Nothing in the scratch has to start at zero: the attention kernel writes every record and every partial slot that
  // the merge reads in the same call, and the merge never touches a slot whose weight is zero.
  return run_decode(q, k, v, k_scale, v_scale, seqlens, block_table, bt_row_stride, 0, 0, out, ws, kStaticScratchBytes, batch,
                    q_len, heads, heads_kv, dim, page_size, n_phys_tokens, q_dtype, kv_dtype, sm_scale, softcap, causal, num_split,
                    kernel, hip_stream);
}

// A contiguous cache is walked in 32-token tiles: the "page size" both kernels do their tile arithmetic with.
static const int kContigTile = 32;

int mi355_gqa_decode_workspace(int batch, int q_len, int heads, int heads_kv, int dim, int64_t max_seqlen_kv, int q_dtype,
                               int kv_dtype, int num_split_in, int kernel, size_t* workspace_bytes, int* num_split_out,
                               int* kernel_out) {
  if (max_seqlen_kv <= 0) return fail(MI355_EINVAL, "max_seqlen_kv must be positive");
  return mi355_gqa_paged_decode_workspace(batch, q_len, heads, heads_kv, dim, kContigTile,
                                          (max_seqlen_kv + kContigTile - 1) / kContigTile, q_dtype, kv_dtype, num_split_in,
                                          kernel, workspace_bytes, num_split_out, kernel_out);
}

int mi355_gqa_decode(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale, void* out,
                     void* workspace, size_t workspace_bytes, int batch, int q_len, int heads, int heads_kv, int dim,
                     int64_t kv_seq_stride, int real_seqlen_kv, int q_dtype, int kv_dtype, float sm_scale, float softcap,
                     int causal, int num_split, int kernel, void* hip_stream) {
  int rc = check_shape(batch, q_len, heads, heads_kv, dim, kContigTile, q_dtype, kv_dtype);
  if (rc) return rc;
  if (batch == 0) return MI355_OK;
  if (!q || !k || !v || !out) return fail(MI355_EINVAL, "q, k, v and out must be non-null");
  if (real_seqlen_kv < 0) return fail(MI355_EINVAL, "real_seqlen_kv must be non-negative, got %d", real_seqlen_kv);
  if (kv_seq_stride <= 0 || kv_seq_stride < real_seqlen_kv)
    return fail(MI355_EINVAL, "kv_seq_stride (%lld) must be positive and at least real_seqlen_kv (%d)",
                (long long)kv_seq_stride, real_seqlen_kv);
  const int64_t max_blocks = ((int64_t)real_seqlen_kv + kContigTile - 1) / kContigTile;
  return run_decode(q, k, v, k_scale, v_scale, nullptr, nullptr, max_blocks > 0 ? max_blocks : 1, kv_seq_stride,
                    real_seqlen_kv, out, workspace, workspace_bytes, batch, q_len, heads, heads_kv, dim, kContigTile,
                    (int64_t)batch * kv_seq_stride, q_dtype, kv_dtype, sm_scale, softcap, causal, num_split, kernel,
                    hip_stream);
}

// Prefill chunk: the workspace holds the decode workspace (shared by the two runs of the fp8 path) and, for an
// fp8 cache, two sets of fp32 rows + LSE.
static size_t prefill_final_bytes(int64_t total_q, int heads, int dim) {
  return align256((size_t)total_q * heads * dim * sizeof(float)) + align256((size_t)total_q * heads * sizeof(float));
}

static int prefill_plans(int batch, int max_seqlen_q, int heads, int heads_kv, int dim, int page_size,
                         int64_t max_pages_per_req, int q_dtype, int cache_dtype, int kernel, Plan* cache_plan, Plan* chunk_plan) {
  int rc = make_plan(batch, max_seqlen_q, heads, heads_kv, dim, page_size, max_pages_per_req, q_dtype, cache_dtype, 0.f, 0,
                     kernel, cache_plan);
  if (rc) return rc;
  *chunk_plan = Plan();
  if (cache_dtype == MI355_DT_FP8_E4M3FN)  // the chunk's own 16-bit tokens are a second, contiguous key set
    rc = make_plan(batch, max_seqlen_q, heads, heads_kv, dim, kContigTile, ((int64_t)max_seqlen_q + kContigTile - 1) / kContigTile,
                   q_dtype, q_dtype, 0.f, 0, kernel, chunk_plan);
  return rc;
}

// FP8 cache with long chunks: instead of one pass over the fp8 pages and one over the chunk, the cached tokens are
// dequantised once into contiguous 16-bit rows (dequant_pack_chunk_kernel), the chunk's tokens copied behind them, and the
// 16-bit kernel makes one pass over both.  Converting in the attention kernel costs every wave that reads a tile its own
// conversion (8 x 512-token chunks on 4 K prefixes: 448 us + 80 us for the chunk against 405 us for the one 16-bit pass);
// converting once costs the cache's bytes five times over (read 1, write 2, read 2), which only pays while the attention
// is compute-bound: from kPackMinRows query rows per kv head, on the MFMA kernel, within kPackMaxBytes of workspace
// (a block table as wide as the whole pool asks for more and keeps the two passes).
constexpr int kPackMinRows = 1024;
constexpr size_t kPackMaxBytes = (size_t)4 << 30;
struct PackPlan {
  bool use = false;
  int stride = 0;          // token rows per sequence slot
  size_t starts_bytes = 0; // kv_starts[batch]
  size_t kv_bytes = 0;     // one of the two packed tensors
  Plan attn;               // the single 16-bit pass
};

static int fp8_prefill_pack_plan(int batch, int max_seqlen_q, int heads, int heads_kv, int dim, int page_size,
                                 int64_t max_pages_per_req, int q_dtype, int kernel, PackPlan* pp) {
  *pp = PackPlan();
  if ((kernel & 0xFF) == MI355_KERNEL_GENERIC) return MI355_OK;
  if ((int64_t)max_seqlen_q * (heads / heads_kv) < kPackMinRows) return MI355_OK;
  const int64_t stride = (max_pages_per_req * page_size + kContigTile - 1) / kContigTile * kContigTile;
  if (stride <= 0 || stride * batch >= INT_MAX) return MI355_OK;
  const size_t kv_bytes = align256((size_t)batch * stride * heads_kv * dim * 2);
  if (2 * kv_bytes > kPackMaxBytes) return MI355_OK;
  int rc = make_plan(batch, max_seqlen_q, heads, heads_kv, dim, kContigTile, stride / kContigTile, q_dtype, q_dtype, 0.f, 0, kernel,
                     &pp->attn);
  if (rc) return rc;
  if (pp->attn.kernel != MI355_KERNEL_MFMA) return MI355_OK;
  pp->use = true;
  pp->stride = (int)stride;
  pp->starts_bytes = align256((size_t)batch * sizeof(int32_t));
  pp->kv_bytes = kv_bytes;
  return MI355_OK;
}

int mi355_gqa_prefill_paged_workspace(int batch, int max_seqlen_q, int64_t total_q, int heads, int heads_kv, int dim,
                                      int page_size, int64_t max_pages_per_req, int q_dtype, int cache_dtype, int kernel,
                                      size_t* workspace_bytes) {
  int rc = check_shape(batch, max_seqlen_q, heads, heads_kv, dim, page_size, q_dtype, cache_dtype);
  if (rc) return rc;
  if (total_q < 0) return fail(MI355_EINVAL, "total_q must be non-negative");
  if (cache_dtype == MI355_DT_FP8_E4M3FN) {
    PackPlan pp;
    rc = fp8_prefill_pack_plan(batch, max_seqlen_q, heads, heads_kv, dim, page_size, max_pages_per_req, q_dtype, kernel, &pp);
    if (rc) return rc;
    if (pp.use) {
      if (workspace_bytes) *workspace_bytes = align256(pp.attn.part_o_bytes + pp.attn.part_lse_bytes) + pp.starts_bytes + 2 * pp.kv_bytes;
      return MI355_OK;
    }
  }
  Plan a, b;
  rc = prefill_plans(batch, max_seqlen_q, heads, heads_kv, dim, page_size, max_pages_per_req, q_dtype, cache_dtype, kernel, &a, &b);
  if (rc) return rc;
  size_t wa = a.part_o_bytes + a.part_lse_bytes, wb = b.part_o_bytes + b.part_lse_bytes;
  size_t total = wa > wb ? wa : wb;
  if (cache_dtype == MI355_DT_FP8_E4M3FN) total += 2 * prefill_final_bytes(total_q, heads, dim);
  if (workspace_bytes) *workspace_bytes = total;
  return MI355_OK;
}

int mi355_gqa_prefill_paged(const void* q, const void* k_new, const void* v_new, void* k_pages, void* v_pages,
                            const float* k_scale, const float* v_scale, const int32_t* cu_seqlens_q,
                            const int32_t* cache_seqlens, const int32_t* block_table, int64_t bt_row_stride, void* out,
                            void* workspace, size_t workspace_bytes, int batch, int max_seqlen_q, int64_t total_q, int heads,
                            int heads_kv, int dim, int page_size, int64_t n_phys_tokens, int q_dtype, int cache_dtype,
                            float sm_scale, float softcap, int causal, int kernel, void* hip_stream) {
  int rc = check_shape(batch, max_seqlen_q, heads, heads_kv, dim, page_size, q_dtype, cache_dtype);
  if (rc) return rc;
  if (batch == 0 || total_q == 0) return MI355_OK;
  if (total_q < 0) return fail(MI355_EINVAL, "total_q must be non-negative");
  if (!q || !k_new || !v_new || !k_pages || !v_pages || !cu_seqlens_q || !cache_seqlens || !block_table || !out)
    return fail(MI355_EINVAL, "q, k_new, v_new, k_pages, v_pages, cu_seqlens_q, cache_seqlens, block_table and out must be non-null");
  const bool fp8 = cache_dtype == MI355_DT_FP8_E4M3FN;
  if (fp8 && (!k_scale || !v_scale)) return fail(MI355_EINVAL, "k_scale and v_scale are required with an fp8 KV cache");
  if (n_phys_tokens <= 0 || n_phys_tokens % page_size != 0)
    return fail(MI355_EINVAL, "n_phys_tokens (%lld) must be a positive multiple of page_size (%d)", (long long)n_phys_tokens, page_size);
  if (bt_row_stride <= 0) return fail(MI355_EINVAL, "bt_row_stride must be positive");
  if (((uintptr_t)k_new | (uintptr_t)v_new | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15)
    return fail(MI355_EINVAL, "k_new, v_new, k_pages and v_pages must be 16-byte aligned");
  size_t need = 0;
  rc = mi355_gqa_prefill_paged_workspace(batch, max_seqlen_q, total_q, heads, heads_kv, dim, page_size, bt_row_stride, q_dtype,
                                         cache_dtype, kernel, &need);
  if (rc) return rc;
  if (need > 0) {
    if (!workspace) return fail(MI355_EWORKSPACE, "workspace of %zu bytes required, got null", need);
    if (workspace_bytes < need) return fail(MI355_EWORKSPACE, "workspace of %zu bytes required, got %zu", need, workspace_bytes);
    if ((uintptr_t)workspace & 255) return fail(MI355_EWORKSPACE, "workspace must be 256-byte aligned");
  }
  rc = check_device();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)hip_stream;
  const char* err = launch_kv_append_chunk(k_new, v_new, k_pages, v_pages, k_scale, v_scale, cu_seqlens_q, cache_seqlens,
                                           block_table, bt_row_stride, batch, total_q, heads_kv, dim, page_size,
                                           n_phys_tokens / page_size, q_dtype, cache_dtype, s);
  if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
  Extras ex;
  ex.cu_q = cu_seqlens_q;
  if (fp8) {
    PackPlan pp;
    rc = fp8_prefill_pack_plan(batch, max_seqlen_q, heads, heads_kv, dim, page_size, bt_row_stride, q_dtype, kernel, &pp);
    if (rc) return rc;
    if (pp.use) {
      const size_t attn_bytes = align256(pp.attn.part_o_bytes + pp.attn.part_lse_bytes);
      int32_t* starts = (int32_t*)((char*)workspace + attn_bytes);
      void* kp = (char*)workspace + attn_bytes + pp.starts_bytes;
      void* vp = (char*)kp + pp.kv_bytes;
      err = launch_dequant_pack_chunk(k_pages, v_pages, k_new, v_new, k_scale, v_scale, cu_seqlens_q, cache_seqlens, block_table,
                                      bt_row_stride, kp, vp, starts, batch, heads_kv, dim, page_size, n_phys_tokens / page_size,
                                      pp.stride, q_dtype, s);
      if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
      ex.len_excludes_new = 1;
      ex.kv_starts = starts;
      return run_decode(q, kp, vp, nullptr, nullptr, cache_seqlens, nullptr, pp.stride / kContigTile, 0, 0, out, workspace, attn_bytes,
                        batch, max_seqlen_q, heads, heads_kv, dim, kContigTile, (int64_t)batch * pp.stride, q_dtype, q_dtype, sm_scale,
                        softcap, causal, 0, kernel, hip_stream, ex);
    }
  }
  if (!fp8) {
    // 16-bit cache: the chunk is in the pages now, bit for bit; one pass over (old + new) tokens
    ex.len_excludes_new = 1;
    return run_decode(q, k_pages, v_pages, nullptr, nullptr, cache_seqlens, block_table, bt_row_stride, 0, 0, out, workspace,
                      workspace_bytes, batch, max_seqlen_q, heads, heads_kv, dim, page_size, n_phys_tokens, q_dtype,
                      cache_dtype, sm_scale, softcap, causal, 0, kernel, hip_stream, ex);
  }
  // fp8 cache: the old tokens come dequantised from the pages (every query sees all of them), the chunk's own tokens
  // unquantised from k_new / v_new (causal inside the chunk) -- gqa_fwd.py:1180-1245 -- and the two results are merged.
  const size_t fin = prefill_final_bytes(total_q, heads, dim);
  const size_t o_bytes = align256((size_t)total_q * heads * dim * sizeof(float));
  char* tail = (char*)workspace + (need - 2 * fin);
  float* o_a = (float*)tail;
  float* lse_a = (float*)(tail + o_bytes);
  float* o_b = (float*)(tail + fin);
  float* lse_b = (float*)(tail + fin + o_bytes);
  ex.scale_per_tensor = 1;
  ex.final_o = o_a;
  ex.final_lse = lse_a;
  rc = run_decode(q, k_pages, v_pages, k_scale, v_scale, cache_seqlens, block_table, bt_row_stride, 0, 0, out, workspace,
                  need - 2 * fin, batch, max_seqlen_q, heads, heads_kv, dim, page_size, n_phys_tokens, q_dtype, cache_dtype,
                  sm_scale, softcap, 0, 0, kernel, hip_stream, ex);
  if (rc) return rc;
  Extras eb;
  eb.cu_q = cu_seqlens_q;
  eb.len_excludes_new = 1;  // with no seqlens array: length = the chunk's own length
  eb.kv_starts = cu_seqlens_q;
  // When the second pass runs on the MFMA kernel it starts every row from the first pass's result and writes the
  // output itself; otherwise it leaves a second fp32 result and merge_two_kernel joins the two.
  Plan plan_a, plan_b;
  rc = prefill_plans(batch, max_seqlen_q, heads, heads_kv, dim, page_size, bt_row_stride, q_dtype, cache_dtype, kernel, &plan_a, &plan_b);
  if (rc) return rc;
  const bool carried = plan_b.kernel == MI355_KERNEL_MFMA;
  if (carried) {
    eb.init_o = o_a;
    eb.init_lse = lse_a;
  } else {
    eb.final_o = o_b;
    eb.final_lse = lse_b;
  }
  rc = run_decode(q, k_new, v_new, nullptr, nullptr, nullptr, nullptr, ((int64_t)max_seqlen_q + kContigTile - 1) / kContigTile, 0, 0,
                  out, workspace, need - 2 * fin, batch, max_seqlen_q, heads, heads_kv, dim, kContigTile,
                  ((total_q + kContigTile - 1) / kContigTile) * kContigTile, q_dtype, q_dtype, sm_scale, softcap, causal, 0, kernel,
                  hip_stream, eb);
  if (rc) return rc;
  if (carried) return MI355_OK;
  err = launch_merge_two(o_a, lse_a, o_b, lse_b, out, total_q * heads, dim, q_dtype, s);
  if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
  return MI355_OK;
}

int mi355_gqa_prefill_paged_rope_workspace(int batch, int max_seqlen_q, int64_t total_q, int heads, int heads_kv, int dim,
                                           int page_size, int64_t max_pages_per_req, int q_dtype, int kernel,
                                           size_t* workspace_bytes) {
  size_t base = 0;
  int rc = mi355_gqa_prefill_paged_workspace(batch, max_seqlen_q, total_q, heads, heads_kv, dim, page_size, max_pages_per_req,
                                             q_dtype, q_dtype, kernel, &base);
  if (rc) return rc;
  // the rotated queries follow the attention workspace
  if (workspace_bytes) *workspace_bytes = align256(base) + align256((size_t)total_q * heads * dim * 2);
  return MI355_OK;
}

int mi355_gqa_prefill_paged_rope(const void* q, const void* k_new, const void* v_new, void* k_pages, void* v_pages,
                                 const void* cos_table, const void* sin_table, const int32_t* cu_seqlens_q,
                                 const int32_t* cache_seqlens, const int32_t* block_table, int64_t bt_row_stride, void* out,
                                 void* workspace, size_t workspace_bytes, int batch, int max_seqlen_q, int64_t total_q,
                                 int heads, int heads_kv, int dim, int page_size, int64_t n_phys_tokens, int q_dtype,
                                 int rotary_dim, int64_t max_position, float sm_scale, float softcap, int causal, int kernel,
                                 void* hip_stream) {
  int rc = check_shape(batch, max_seqlen_q, heads, heads_kv, dim, page_size, q_dtype, q_dtype);
  if (rc) return rc;
  if (rotary_dim <= 0 || rotary_dim % 2 != 0 || rotary_dim > dim)
    return fail(MI355_EINVAL, "rotary_dim (%d) must be positive, even, and <= dim (%d)", rotary_dim, dim);
  if (max_position <= 0) return fail(MI355_EINVAL, "max_position must be positive");
  if (batch == 0 || total_q == 0) return MI355_OK;
  if (total_q < 0) return fail(MI355_EINVAL, "total_q must be non-negative");
  if (!q || !k_new || !v_new || !k_pages || !v_pages || !cos_table || !sin_table || !cu_seqlens_q || !cache_seqlens ||
      !block_table || !out)
    return fail(MI355_EINVAL, "q, k_new, v_new, k_pages, v_pages, cos_table, sin_table, cu_seqlens_q, cache_seqlens, block_table and out must be non-null");
  if (n_phys_tokens <= 0 || n_phys_tokens % page_size != 0)
    return fail(MI355_EINVAL, "n_phys_tokens (%lld) must be a positive multiple of page_size (%d)", (long long)n_phys_tokens, page_size);
  if (bt_row_stride <= 0) return fail(MI355_EINVAL, "bt_row_stride must be positive");
  if (((uintptr_t)q | (uintptr_t)k_new | (uintptr_t)v_new | (uintptr_t)k_pages | (uintptr_t)v_pages | (uintptr_t)cos_table |
       (uintptr_t)sin_table) & 15)
    return fail(MI355_EINVAL, "q, k_new, v_new, k_pages, v_pages, cos_table and sin_table must be 16-byte aligned");
  size_t base = 0, need = 0;
  rc = mi355_gqa_prefill_paged_workspace(batch, max_seqlen_q, total_q, heads, heads_kv, dim, page_size, bt_row_stride, q_dtype,
                                         q_dtype, kernel, &base);
  if (rc) return rc;
  rc = mi355_gqa_prefill_paged_rope_workspace(batch, max_seqlen_q, total_q, heads, heads_kv, dim, page_size, bt_row_stride,
                                              q_dtype, kernel, &need);
  if (rc) return rc;
  if (!workspace) return fail(MI355_EWORKSPACE, "workspace of %zu bytes required, got null", need);
  if (workspace_bytes < need) return fail(MI355_EWORKSPACE, "workspace of %zu bytes required, got %zu", need, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(MI355_EWORKSPACE, "workspace must be 256-byte aligned");
  rc = check_device();
  if (rc) return rc;
  void* q_rot = (char*)workspace + align256(base);
  const char* err = launch_rope_append_chunk(q, k_new, v_new, q_rot, k_pages, v_pages, cos_table, sin_table, cu_seqlens_q,
                                             cache_seqlens, block_table, bt_row_stride, batch, total_q, heads, heads_kv, dim,
                                             rotary_dim, max_position, page_size, n_phys_tokens / page_size, q_dtype,
                                             (hipStream_t)hip_stream);
  if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
  // the rotated chunk is in the pages now: one pass over (old + new) tokens with the rotated queries
  Extras ex;
  ex.cu_q = cu_seqlens_q;
  ex.len_excludes_new = 1;
  return run_decode(q_rot, k_pages, v_pages, nullptr, nullptr, cache_seqlens, block_table, bt_row_stride, 0, 0, out, workspace,
                    align256(base), batch, max_seqlen_q, heads, heads_kv, dim, page_size, n_phys_tokens, q_dtype, q_dtype,
                    sm_scale, softcap, causal, 0, kernel, hip_stream, ex);
}

int mi355_gather_probe(const void* cache, const int32_t* seqlens, const int32_t* block_table, int64_t bt_row_stride,
                       void* dense_out, int batch, int64_t max_len, int64_t row_bytes, int page_size, int64_t n_phys_tokens,
                       void* hip_stream) {
  if (batch < 0 || max_len < 0) return fail(MI355_EINVAL, "batch and max_len must be non-negative");
  if (batch > 65535) return fail(MI355_EUNSUPPORTED, "batch %d exceeds 65535", batch);
  if (page_size <= 0) return fail(MI355_EINVAL, "page_size must be positive");
  if (row_bytes <= 0 || row_bytes % 4 != 0) return fail(MI355_EINVAL, "row_bytes must be a positive multiple of 4");
  if (n_phys_tokens <= 0 || n_phys_tokens % page_size != 0)
    return fail(MI355_EINVAL, "n_phys_tokens must be a positive multiple of page_size");
  if (bt_row_stride <= 0) return fail(MI355_EINVAL, "bt_row_stride must be positive");
  if (batch == 0 || max_len == 0) return MI355_OK;
  if (!cache || !seqlens || !block_table || !dense_out) return fail(MI355_EINVAL, "null pointer argument");
  if (int rc = check_device()) return rc;
  const char* err = launch_gather_probe(cache, seqlens, block_table, bt_row_stride, dense_out, batch, max_len, row_bytes,
                                        page_size, n_phys_tokens / page_size, (hipStream_t)hip_stream);
  if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
  return MI355_OK;
}

int mi355_kv_append_fp8(const void* x_new, void* cache, float* scale, const int32_t* seqlens, const int32_t* block_table,
                        int64_t bt_row_stride, int batch, int heads_kv, int dim, int page_size, int64_t n_phys_tokens,
                        int x_dtype, void* hip_stream) {
  if (batch < 0 || batch > 65535) return fail(MI355_EINVAL, "batch must be in [0, 65535]");
  if (heads_kv <= 0) return fail(MI355_EINVAL, "heads_kv must be positive");
  if (dim != 64 && dim != 128 && dim != 256) return fail(MI355_EUNSUPPORTED, "head dim %d is not served (64, 128 or 256)", dim);
  if (page_size <= 0) return fail(MI355_EINVAL, "page_size must be positive");
  if (!is_q_dtype(x_dtype)) return fail(MI355_EINVAL, "x_dtype must be bf16 or fp16");
  if (n_phys_tokens <= 0 || n_phys_tokens % page_size != 0)
    return fail(MI355_EINVAL, "n_phys_tokens must be a positive multiple of page_size");
  if (bt_row_stride <= 0) return fail(MI355_EINVAL, "bt_row_stride must be positive");
  if (batch == 0) return MI355_OK;
  if (!x_new || !cache || !scale || !seqlens || !block_table) return fail(MI355_EINVAL, "null pointer argument");
  if (int rc = check_device()) return rc;
  const char* err = launch_kv_append_fp8(x_new, cache, scale, seqlens, block_table, bt_row_stride, batch, heads_kv, dim,
                                         page_size, n_phys_tokens / page_size, x_dtype, (hipStream_t)hip_stream);
  if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
  return MI355_OK;
}

int mi355_prefill_input_facts(const int32_t* cu_seqlens_q, const int32_t* cache_seqlens, const int32_t* block_table,
                              int64_t bt_row_stride, const float* k_scale, const float* v_scale, int batch, int max_pages_per_req,
                              int32_t* facts, void* hip_stream) {
  if (batch <= 0 || max_pages_per_req <= 0) return fail(MI355_EINVAL, "batch and max_pages_per_req must be positive");
  if (bt_row_stride < max_pages_per_req) return fail(MI355_EINVAL, "bt_row_stride must be at least max_pages_per_req");
  if (!cu_seqlens_q || !cache_seqlens || !block_table || !facts) return fail(MI355_EINVAL, "null pointer argument");
  if (int rc = check_device()) return rc;
  const char* err = launch_prefill_input_facts(cu_seqlens_q, cache_seqlens, block_table, bt_row_stride, k_scale, v_scale, batch,
                                               max_pages_per_req, facts, (hipStream_t)hip_stream);
  if (err) return fail(MI355_ELAUNCH, "kernel launch failed: %s", err);
  return MI355_OK;
}

}  // extern "C"
