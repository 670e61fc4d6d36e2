// Runtime (client, device, buffers, executables, futures) and the C ABI declared
// in include/reactant_mi355x.h.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hiprtc.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <unordered_set>
#include <vector>

#include "../../include/reactant_mi355x.h"
#include "rx_embedded.inc"
#include "rx_ir.h"
#include "rx_plan.h"
#include "rx_gemm.h"

#define RX_EXPORT extern "C" __attribute__((visibility("default")))

extern "C" __attribute__((visibility("default"))) void (*ReactantThrowError)(const char*) = nullptr;

// Device memory of RxExecuteNoAlloc: every temporary of an executable's plan (partial results of the
// two-pass reductions, intermediate tensors between kernels) is placed here instead of coming from
// the allocator.  One copy per GPU, held until the process ends.  Host code never uses this name as
// an address: each device's address is looked up once (hipGetSymbolAddress, in MakeGPUClient) and
// kept in RxDevice::scratch_ptr.
#define RX_NOALLOC_SCRATCH_BYTES (4u << 20)
static __device__ __align__(256) unsigned char scratch[RX_NOALLOC_SCRATCH_BYTES];

namespace {

using rx::Error;

thread_local std::string g_last_error;

void report_error(const std::string& msg) {
  g_last_error = msg;
  if (ReactantThrowError) ReactantThrowError(msg.c_str());
}

#define HIP_CHECK(expr)                                                                                   \
  do {                                                                                                    \
    hipError_t e_ = (expr);                                                                               \
    if (e_ != hipSuccess) throw Error(std::string(#expr) + " failed: " + hipGetErrorString(e_));          \
  } while (0)

char* dup_cstr(const std::string& s) {
  char* p = (char*)malloc(s.size() + 1);
  memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

// ---------------------------------------------------------------------------
// handle registry
// ---------------------------------------------------------------------------
std::mutex g_reg_mu;
std::unordered_set<const void*> g_handles;
void reg_add(const void* p) { std::lock_guard<std::mutex> l(g_reg_mu); g_handles.insert(p); }
void reg_del(const void* p) { std::lock_guard<std::mutex> l(g_reg_mu); g_handles.erase(p); }
bool reg_has(const void* p) { std::lock_guard<std::mutex> l(g_reg_mu); return g_handles.count(p) != 0; }

}  // namespace

// ---------------------------------------------------------------------------
// objects behind the opaque handles
// ---------------------------------------------------------------------------
struct RxClient;

struct RxDevice {
  RxClient* client = nullptr;
  int ordinal = 0;       // HIP device ordinal
  int index = 0;         // position in the client's device list
  hipStream_t stream = nullptr;
  void* scratch_ptr = nullptr;   // this device's copy of `scratch` (RxExecuteNoAlloc)
  // A word in pinned host memory that kernels can write: set when a kernel's bounded wait for another workgroup of
  // its launch expired (its results are then invalid).  Checked wherever the host has waited for the device.
  unsigned* fault_host = nullptr;
  void* fault_dev = nullptr;
  // set once the fault word has been found set: executables whose kernels wait for other workgroups are then rebuilt
  // in the form that does not wait, and new ones are compiled in that form
  std::atomic<bool> waits_failed{false};
  std::mutex scratch_mu;         // held while a call that uses it queues its kernels
  std::mutex future_mu;          // held while a future of this device creates and records its event
  std::string kind;
  std::string arch;
  // caching allocator: device memory is kept and reused by size class, because hipMalloc and
  // hipFree are slow and hipFree synchronizes.  All work of a device runs on one stream, so
  // a block freed by the host may be handed out again immediately: stream order protects it.
  std::mutex mu;
  std::multimap<size_t, void*> free_blocks;
  int64_t num_allocs = 0, bytes_in_use = 0, peak_bytes_in_use = 0, largest_alloc = 0, pool_bytes = 0, peak_pool_bytes = 0;
  int64_t bytes_limit = 0;

  static size_t round_size(size_t n) {
    if (n == 0) n = 1;
    if (n <= (1u << 20)) return (n + 255) & ~(size_t)255;
    return (n + 65535) & ~(size_t)65535;
  }
  void* alloc(size_t n) {
    const size_t r = round_size(n);
    std::lock_guard<std::mutex> l(mu);
    auto it = free_blocks.find(r);
    void* p = nullptr;
    if (it != free_blocks.end()) {
      p = it->second;
      free_blocks.erase(it);
    } else {
      HIP_CHECK(hipSetDevice(ordinal));
      auto trim = [&] {   // give cached blocks back to the driver
        for (auto& kv : free_blocks) { (void)hipFree(kv.second); pool_bytes -= (int64_t)kv.first; }
        free_blocks.clear();
      };
      // the client's memory fraction bounds what this allocator holds, cached blocks included
      if (bytes_limit > 0 && pool_bytes + (int64_t)r > bytes_limit) {
        trim();
        if (pool_bytes + (int64_t)r > bytes_limit)
          throw Error("RESOURCE_EXHAUSTED: allocating " + std::to_string(r) + " bytes would exceed the client's memory limit of " +
                      std::to_string(bytes_limit) + " bytes (" + std::to_string(pool_bytes) + " in use)");
      }
      hipError_t e = hipMalloc(&p, r);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        trim();
        e = hipMalloc(&p, r);
        if (e != hipSuccess) {
          (void)hipGetLastError();
          throw Error("RESOURCE_EXHAUSTED: out of device memory allocating " + std::to_string(r) + " bytes (" + hipGetErrorString(e) + ")");
        }
      }
      pool_bytes += (int64_t)r;
      peak_pool_bytes = std::max(peak_pool_bytes, pool_bytes);
    }
    num_allocs++;
    bytes_in_use += (int64_t)r;
    peak_bytes_in_use = std::max(peak_bytes_in_use, bytes_in_use);
    largest_alloc = std::max<int64_t>(largest_alloc, (int64_t)r);
    return p;
  }
  bool closed = false;   // the client is gone: nothing will ask for a cached block again
  void release(void* p, size_t n) {
    const size_t r = round_size(n);
    std::lock_guard<std::mutex> l(mu);
    bytes_in_use -= (int64_t)r;
    if (closed) {   // a buffer freed late (a finalizer after FreeClient): hand the block straight back
      (void)hipSetDevice(ordinal);
      (void)hipFree(p);
      pool_bytes -= (int64_t)r;
      return;
    }
    free_blocks.insert({r, p});
  }
  void drain(bool close) {
    std::lock_guard<std::mutex> l(mu);
    for (auto& kv : free_blocks) { (void)hipFree(kv.second); pool_bytes -= (int64_t)kv.first; }
    free_blocks.clear();
    closed = closed || close;
  }
};

struct Allocation {
  RxDevice* dev;
  void* ptr;
  size_t bytes;
  Allocation(RxDevice* d, size_t n) : dev(d), ptr(d->alloc(n)), bytes(n) {}
  ~Allocation() { dev->release(ptr, bytes); }
  Allocation(const Allocation&) = delete;
};
using Mem = std::shared_ptr<Allocation>;

struct RxClient {
  std::vector<std::unique_ptr<RxDevice>> devices;
  std::atomic<bool> alive{true};
};

struct RxBuffer {
  RxClient* client = nullptr;
  RxDevice* device = nullptr;
  Mem mem;                       // empty once donated
  rx::TType ty;
  bool donated = false;
};

struct RxFuture {
  hipEvent_t ev = nullptr;       // recorded when the future is first asked (future_event)
  bool done = false;             // known complete without an event (its client was freed, which waits for the stream)
  RxDevice* device = nullptr;
  std::string error;
};

// Called after the host has waited for a device: a kernel whose wait for another workgroup expired has set the word.
static void check_fault(RxDevice* d) {
  if (!d || !d->fault_host) return;
  volatile unsigned* w = d->fault_host;
  if (*w == 0) return;
  *w = 0;
  d->waits_failed = true;
  throw Error("INTERNAL: a kernel's bounded wait for another workgroup of its launch expired; results produced since the last "
              "synchronization are invalid.  Executables of this device that wait between workgroups (the one-launch scan) are "
              "rebuilt in the form that does not wait when they are next executed, so the call can be repeated");
}

struct RxExecutable {
  RxClient* client = nullptr;
  RxDevice* device = nullptr;
  rx::Plan plan;
  hipModule_t module = nullptr;
  std::vector<hipFunction_t> fns;   // per launch
  std::vector<Mem> consts;          // per plan buffer (only Const kinds are set)
  std::string report;
  std::string text;                 // the module as compiled: a rebuild after a failed wait starts from it
  bool waits = false;               // some kernel of the plan waits for other workgroups of its launch (has a fault-word argument)
  std::mutex mu;
  // event lists of executions profiled without blocking (RxExecuteProfiled), oldest first
  std::vector<std::vector<hipEvent_t>> pending_events;
};

namespace {

// ---------------------------------------------------------------------------
// hiprtc
// ---------------------------------------------------------------------------
std::string rtc_compile(const std::string& source, const std::string& arch) {
  hiprtcProgram prog;
  const char* hdr_src[] = {kRxPreambleSrc, kRxGemmKernelsSrc};
  const char* hdr_name[] = {"rx_preamble.h", "rx_gemm_kernels.h"};
  hiprtcResult r = hiprtcCreateProgram(&prog, source.c_str(), "rx_module.hip", 2, hdr_src, hdr_name);
  if (r != HIPRTC_SUCCESS) throw Error(std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
  std::string archopt = "--offload-arch=" + arch;
  std::vector<const char*> opts = {archopt.c_str(), "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
                                   "-packed-fp32-ops", "-Wno-unused-value"};
  r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
  size_t ls = 0;
  hiprtcGetProgramLogSize(prog, &ls);
  std::string log(ls, '\0');
  if (ls) hiprtcGetProgramLog(prog, &log[0]);
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    if (getenv("RX_DUMP_FAILED_SOURCE")) {
      FILE* f = fopen(getenv("RX_DUMP_FAILED_SOURCE"), "w");
      if (f) { fputs(source.c_str(), f); fclose(f); }
    }
    throw Error(std::string("kernel compilation failed (") + hiprtcGetErrorString(r) + "):\n" + log);
  }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  std::string code(cs, '\0');
  hiprtcGetCode(prog, &code[0]);
  hiprtcDestroyProgram(&prog);
  return code;
}

rx::PlanOptions plan_options() {
  rx::PlanOptions o;
  if (const char* e = getenv("RX_XCD_SLABS")) o.xcd_slabs = atoi(e) != 0;
  if (const char* e = getenv("RX_SLAB_MIN_NUMEL")) o.slab_min_numel = o.slab_order_min_numel = atoll(e);
  if (const char* e = getenv("RX_SLAB_ORDER_MIN_NUMEL")) o.slab_order_min_numel = atoll(e);
  if (const char* e = getenv("RX_MFMA")) o.mfma = atoi(e) != 0;
  if (const char* e = getenv("RX_ROW_FUSION")) o.row_fusion = atoi(e) != 0;
  if (const char* e = getenv("RX_LDS_STENCIL")) o.lds_stencil = atoi(e) != 0;
  if (const char* e = getenv("RX_STENCIL_MARCH2")) o.stencil_march2 = atoi(e) != 0;
  if (const char* e = getenv("RX_TRANSPOSE_VECTORS")) o.transpose_vectors = atoi(e) != 0;
  if (const char* e = getenv("RX_TRANSPOSE_BLOCK")) o.transpose_block = std::max(1, std::min(64, atoi(e)));
  if (const char* e = getenv("RX_MARCH2_PREFETCH")) o.march2_prefetch = atoi(e) == 2 ? 2 : 1;
  if (const char* e = getenv("RX_MARCH2_EDGE")) o.march2_edge = atoi(e) != 0;
  if (const char* e = getenv("RX_MARCH2_LDS_BALLAST")) o.march2_lds_ballast = std::max(0, atoi(e));
  if (const char* e = getenv("RX_MARCH2_PLANES")) o.march2_planes = atoi(e) > 0 ? atoi(e) : o.march2_planes;
  if (const char* e = getenv("RX_MARCH2_TILE")) { int v[2]; if (sscanf(e, "%d,%d", &v[0], &v[1]) == 2) { o.march2_tile[0] = v[0]; o.march2_tile[1] = v[1]; } }
  if (const char* e = getenv("RX_LDS_TILE")) { int v[3]; if (sscanf(e, "%d,%d,%d", &v[0], &v[1], &v[2]) == 3) { o.lds_tile[0] = v[0]; o.lds_tile[1] = v[1]; o.lds_tile[2] = v[2]; } }
  if (const char* e = getenv("RX_LDS_TILE2")) { int v[3]; if (sscanf(e, "%d,%d,%d", &v[0], &v[1], &v[2]) == 3) { o.lds_tile2[0] = v[0]; o.lds_tile2[1] = v[1]; o.lds_tile2[2] = v[2]; } }
  if (const char* e = getenv("RX_SLAB_YTILES")) o.slab_ytiles = atoi(e);
  if (const char* e = getenv("RX_LDS2_THREADS")) o.lds2_threads = atoi(e);
  if (const char* e = getenv("RX_SINGLE_PASS_REDUCE")) o.single_pass_reduce = atoi(e) != 0;
  if (const char* e = getenv("RX_SINGLE_PASS_SCAN")) o.single_pass_scan = atoi(e) != 0;
  if (const char* e = getenv("RX_LDS_TRANSPOSE")) o.lds_transpose = atoi(e) != 0;
  if (const char* e = getenv("RX_DOT_AS_REDUCE")) o.dot_as_reduce = atoi(e) != 0;
  if (const char* e = getenv("RX_FUSE_DOT_OPERANDS")) o.fuse_dot_operands = atoi(e) != 0;
  if (const char* e = getenv("RX_BRANCHLESS")) o.branchless_guards = atoi(e) != 0;
  if (const char* e = getenv("RX_CLAMP_PADS")) o.clamp_pad_reads = atoi(e) != 0;
  if (const char* e = getenv("RX_TRANSPOSE_OFFSETS")) o.transpose_offsets = atoi(e) != 0;
  if (const char* e = getenv("RX_STENCIL_FUSE")) o.stencil_fuse_steps = atoi(e) != 0;
  if (const char* e = getenv("RX_SPLIT_K")) o.split_k = atoi(e) != 0;
  if (const char* e = getenv("RX_WINDOW_VECTORS")) o.window_reduce_vectors = atoi(e) != 0;
  if (const char* e = getenv("RX_CONV_TAILS")) o.conv_tails = atoi(e);
  if (const char* e = getenv("RX_NHWC_POOLS")) o.nhwc_pools = atoi(e) != 0;
  if (const char* e = getenv("RX_MERGE_MAPS")) o.merge_parameter_maps = atoi(e) != 0;
  if (const char* e = getenv("RX_REDUCE_ROW_BLOCKS")) o.reduce_row_blocks = atoi(e) != 0;
  if (const char* e = getenv("RX_NHWC_REGIONS")) o.nhwc_regions = atoi(e) != 0;
  if (const char* e = getenv("RX_NHWC_REGION_RATIO")) o.nhwc_region_ratio = atof(e);
  if (const char* e = getenv("RX_PAD_INTO_POOLS")) o.pad_into_pools = atoi(e) != 0;
  if (const char* e = getenv("RX_EPILOGUES")) o.product_epilogues = atoi(e) != 0;
  if (const char* e = getenv("RX_EPILOGUE_INIT")) o.epilogue_init = atoi(e) != 0;
  if (const char* e = getenv("RX_CHAIN_CONVS")) o.chain_convs = atoi(e) != 0;
  if (const char* e = getenv("RX_IN_PLACE")) o.in_place_updates = atoi(e) != 0;
  if (const char* e = getenv("RX_CHAIN_STEPS")) o.chain_steps = atoi(e);
  if (const char* e = getenv("RX_CHAIN_TILE")) { int v[3] = {0, 0, 0}; if (sscanf(e, "%d,%d,%d", &v[0], &v[1], &v[2]) >= 1) { o.chain_tile[0] = v[0]; o.chain_tile[1] = v[1]; o.chain_tile[2] = v[2]; } }
  if (const char* e = getenv("RX_CHAIN_MAX_RANK")) o.chain_max_rank = atoi(e);
  if (const char* e = getenv("RX_CHAIN_FIXED")) o.chain_fixed_cells = atoi(e) != 0;
  if (const char* e = getenv("RX_CHAIN_THREADS")) o.chain_threads = atoi(e);
  if (const char* e = getenv("RX_CHAIN_LDS_BYTES")) o.chain_lds_bytes = atoll(e);
  if (const char* e = getenv("RX_CHAIN_REDUNDANCY")) o.chain_redundancy = atof(e);
  if (const char* e = getenv("RX_SHIFTED_VEC")) o.shifted_vector_loads = atoi(e) != 0;
  if (const char* e = getenv("RX_EXCESS_PRECISION")) o.excess_precision = atoi(e) != 0;
  if (const char* e = getenv("RX_NT_LOADS")) o.nt_loads = atoi(e) != 0;
  if (const char* e = getenv("RX_NT_STORES")) o.nt_stores = atoi(e) != 0;
  return o;
}

int64_t prim_numel(size_t nd, const int64_t* dims) {
  int64_t n = 1;
  for (size_t k = 0; k < nd; ++k) n *= dims[k];
  return n;
}

template <typename F>
auto guarded(F&& f, decltype(f()) fallback) -> decltype(f()) {
  try {
    return f();
  } catch (const std::exception& e) {
    report_error(e.what());
    return fallback;
  }
}
template <typename F>
void guarded_void(F&& f) {
  try {
    f();
  } catch (const std::exception& e) {
    report_error(e.what());
  }
}

void check_client(RxClient* c) { if (!c || !reg_has(c)) throw Error("INVALID_ARGUMENT: null or foreign client handle"); }
void check_device(RxDevice* d) { if (!d || !reg_has(d)) throw Error("INVALID_ARGUMENT: null or foreign device handle"); }
void check_buffer(RxBuffer* b) { if (!b || !reg_has(b)) throw Error("INVALID_ARGUMENT: null or foreign buffer handle"); }
void check_exec(RxExecutable* e) { if (!e || !reg_has(e)) throw Error("INVALID_ARGUMENT: null or foreign executable handle"); }

RxBuffer* new_buffer(RxClient* c, RxDevice* d, const rx::TType& ty, Mem mem) {
  RxBuffer* b = new RxBuffer;
  b->client = c;
  b->device = d;
  b->ty = ty;
  b->mem = std::move(mem);
  reg_add(b);
  return b;
}

// AOT kernels ------------------------------------------------------------------
}  // namespace
#include "kernels/rx_preamble.h"
#include "kernels/rx_gemm_kernels.h"
namespace {
__global__ __launch_bounds__(256) void rx_copy16(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n16; i += stride) dst[i] = src[i];
}

// The rate the MFMA pipe sustains when nothing else runs: every wavefront of the chip (one per SIMD) issues
// independent MFMAs back to back on operands that stay in registers, for long enough that the clock settles under
// the power limit.  KIND 0: v_mfma_f32_16x16x32_bf16, KIND 1: v_mfma_f32_16x16x128_f8f6f4 (e4m3 x e4m3), the
// instructions of the streaming GEMM skeleton.  Operands are seeded pseudo-random values of moderate exponent, or all zero
// (no toggling in the multipliers).  Every wavefront reports its shader-clock and real-time ticks.
typedef float rx_probe_f32x16 __attribute__((ext_vector_type(16)));
typedef float rx_probe_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 rx_probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef int rx_probe_i32x8 __attribute__((ext_vector_type(8)));
typedef int rx_probe_i32x4 __attribute__((ext_vector_type(4)));
template <int KIND>
__global__ __launch_bounds__(256) void rx_mfma_probe(unsigned long long* ticks, int iters, int zero) {
  const int tid = threadIdx.x;
  rx_probe_i32x8 a[4], b[4];
  unsigned s = (blockIdx.x * 256u + (unsigned)tid) * 2654435761u + 12345u;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      s = s * 1664525u + 1013904223u;
      unsigned x = KIND == 0 ? ((s & 0x807f807fu) | 0x3f003f00u) : (s & 0xbfbfbfbfu);
      a[i][r] = zero ? 0 : (int)x;
      s = s * 1664525u + 1013904223u;
      x = KIND == 0 ? ((s & 0x807f807fu) | 0x3f003f00u) : (s & 0xbfbfbfbfu);
      b[i][r] = zero ? 0 : (int)x;
    }
  rx_probe_bf16x8 av[4], bv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const rx_probe_i32x4 x = {a[i][0], a[i][1], a[i][2], a[i][3]}, y = {b[i][4], b[i][5], b[i][6], b[i][7]};
    av[i] = __builtin_bit_cast(rx_probe_bf16x8, x);
    bv[i] = __builtin_bit_cast(rx_probe_bf16x8, y);
  }
  rx_probe_f32x16 acc[8];
  rx_probe_f32x4 acc4[16];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc4[i] = rx_probe_f32x4{0.f, 0.f, 0.f, 0.f};
  const unsigned long long t0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    if constexpr (KIND == 0) {
      // written as instructions so that the sixteen accumulators stay in the vector registers they start in
#pragma unroll
      for (int q = 0; q < 32; ++q) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc4[q & 15]) : "v"(av[q & 3]), "v"(bv[(q >> 2) & 3]));
    } else {
#pragma unroll
      for (int q = 0; q < 16; ++q) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+v"(acc4[q & 15]) : "v"(a[q & 3]), "v"(b[(q >> 2) & 3]));
    }
  }
  const unsigned long long t1 = clock64(), w1 = wall_clock64();
  float sum = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) sum += acc[i][0] + acc[i][7];
#pragma unroll
  for (int i = 0; i < 16; ++i) sum += acc4[i][0] + acc4[i][3];
  if (sum == 1.2345f) ticks[2 * 1024] = 1;   // keeps the accumulators alive
  if ((tid & 63) == 0) {
    ticks[(blockIdx.x * 4 + (tid >> 6)) * 2] = t1 - t0;
    ticks[(blockIdx.x * 4 + (tid >> 6)) * 2 + 1] = w1 - w0;
  }
}

// The two large GEMM kernels of the benchmark (the 8192 x 4096 x 4096 bf16 layer, operands [m][k] x [k][n], and the
// 8192^3 e4m3 product, [m][k] x [n][k]) as the planner instantiates them, with a plain scaling epilogue and the clock
// probe of rx_gemm_kernels.h: RxGemmClockProbe.
struct rx_probe_epi {
  rx_u16* __restrict__ out;
  int ld;
  template <int NV> __device__ __forceinline__ void operator()(const float (&acc)[NV], int m, int n) const {
    rx_vec<rx_u16, NV> res;
#pragma unroll
    for (int l = 0; l < NV; ++l) res.v[l] = rx_f32_to_bf16(acc[l] * 0.001f);
    *reinterpret_cast<rx_vec<rx_u16, NV>*>(out + (long long)m * ld + n) = res;
  }
};
template <int KIND>
__global__ __launch_bounds__(512) void rx_gemm_clock_probe(const void* __restrict__ A, const void* __restrict__ B, rx_u16* __restrict__ out,
                                                           unsigned long long* __restrict__ sleep_ticks, unsigned long long* __restrict__ life_ticks) {
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  rx_clock_probe probe{sleep_ticks};
  if constexpr (KIND == 2) {
    // the bf16 layer on the ping-pong body, as the planner instantiates it: sleep_ticks takes the phase probe's figures
    rx_probe_epi epi{out, 4096};
    rx_gemm_body_pp<rx_el_bf16, 256, 256, 2, 4, true, false, 8192, 4096, 4096, 4, 8, false, rx_probe_epi, rx_phase_probe>((const rx_u16*)A, (const rx_u16*)B, epi, rx_phase_probe{sleep_ticks});
  } else if constexpr (KIND == 0) {
    rx_probe_epi epi{out, 4096};
    rx_gemm_body_s<rx_el_bf16, 256, 256, 2, 4, true, false, 8192, 4096, 4096, 4, 8, false, rx_probe_epi, 2, 2, rx_clock_probe>((const rx_u16*)A, (const rx_u16*)B, epi, probe);
  } else {
    rx_probe_epi epi{out, 8192};
    rx_gemm_body_s<rx_el_f8, 256, 256, 2, 4, true, true, 8192, 8192, 8192, 4, 8, false, rx_probe_epi, 2, 2, rx_clock_probe>((const rx_u8*)A, (const rx_u8*)B, epi, probe);
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0) { life_ticks[blockIdx.x * 2] = c1 - c0; life_ticks[blockIdx.x * 2 + 1] = r1 - r0; }
}
// Pseudo-random operands shaped like the benchmark's: mode 0 bf16 ~ N(0, 1) (activations), mode 1 bf16 uniform in
// +-0.027 (Glorot weights of a 4096-wide layer), mode 2 e4m3 of N(0, 1) scaled to an absmax of 448 at 5.5 sigma (a tensor
// quantized with a per-tensor scale).  The normal is a sum of four uniforms.
__global__ __launch_bounds__(256) void rx_probe_fill(void* __restrict__ dst, size_t n, int mode, unsigned seed) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n; i += stride) {
    unsigned s = ((unsigned)i + seed) * 2654435761u + 12345u;
    float u[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      s ^= s >> 15; s *= 2246822519u; s ^= s >> 13; s *= 3266489917u; s ^= s >> 16;
      u[k] = (float)(s >> 8) * (1.0f / 16777216.0f);
    }
    const float g = (u[0] + u[1] + u[2] + u[3] - 2.0f) * 1.7320508f;   // variance 4 / 12 -> 1
    if (mode == 0) ((rx_u16*)dst)[i] = rx_f32_to_bf16(g);
    else if (mode == 1) ((rx_u16*)dst)[i] = rx_f32_to_bf16((u[0] * 2.0f - 1.0f) * 0.027f);
    else ((rx_u8*)dst)[i] = rx_f32_to_e4m3(g * (448.0f / 5.5f));
  }
}

void rebuild_without_waits(RxExecutable* ex);

// Core of XLAExecuteSharded / RxExecuteTimed
void execute(RxExecutable* ex, int num_args, RxBuffer** args, RxDevice* dev, uint8_t* donate, int num_results, RxBuffer** results, float* launch_ms,
             RxFuture** futures, bool profile_async = false) {
  check_exec(ex);
  if (dev) check_device(dev);
  if (!dev) dev = ex->device;
  if (dev != ex->device) throw Error("INVALID_ARGUMENT: executable was compiled for another device");
  std::lock_guard<std::mutex> lock(ex->mu);
  rebuild_without_waits(ex);
  const rx::Plan& P = ex->plan;
  if (num_args != (int)P.param_types.size())
    throw Error("INVALID_ARGUMENT: executable expects " + std::to_string(P.param_types.size()) + " arguments, got " + std::to_string(num_args));
  if (num_results != (int)P.result_types.size())
    throw Error("Error: results.size()=" + std::to_string(P.result_types.size()) + " does not match num_results=" + std::to_string(num_results) + "\n");
  for (int i = 0; i < num_args; ++i) {
    check_buffer(args[i]);
    if (args[i]->donated || !args[i]->mem) throw Error("INVALID_ARGUMENT: argument " + std::to_string(i) + " was donated to an earlier execution");
    if (!(args[i]->ty == P.param_types[i]))
      throw Error("INVALID_ARGUMENT: argument " + std::to_string(i) + " has type " + args[i]->ty.str() + ", executable expects " + P.param_types[i].str());
    if (args[i]->device != dev) throw Error("INVALID_ARGUMENT: argument " + std::to_string(i) + " lives on another device");
  }
  HIP_CHECK(hipSetDevice(dev->ordinal));
  const size_t NB = P.buffers.size();
  std::vector<Mem> bufs(NB);
  std::vector<char> is_res(NB, 0);
  for (int b : P.result_buffers) is_res[b] = 1;
  // A donated argument hands its storage to the plan's buffer now, so that the block goes back to the pool at the
  // argument's last use inside this execution (the time loop of the stencil donates four fields of half a gigabyte).
  // If a later step throws, the guard below gives the storage back where it is still alive; where the plan has already
  // released it, the argument stays consumed.
  struct Donation {
    int num_args;
    RxBuffer** args;
    uint8_t* donate;
    const rx::Plan& P;
    std::vector<Mem>& bufs;
    bool committed = false;
    ~Donation() {
      if (!donate) return;
      for (size_t b = 0; b < P.buffers.size(); ++b) {
        const auto& B = P.buffers[b];
        if (B.kind != rx::BufferDesc::Param || !donate[B.param_index]) continue;
        RxBuffer* a = args[B.param_index];
        if (committed || !bufs[b]) { a->donated = true; a->mem.reset(); }
        else if (!a->mem) a->mem = bufs[b];
      }
    }
  } donation{num_args, args, donate, P, bufs};
  for (size_t b = 0; b < NB; ++b) {
    const auto& B = P.buffers[b];
    if (B.kind == rx::BufferDesc::Param) {
      RxBuffer* a = args[B.param_index];
      bufs[b] = a->mem;
    } else if (B.kind == rx::BufferDesc::Const) {
      bufs[b] = ex->consts[b];
    }
  }
  if (donate)
    for (int i = 0; i < num_args; ++i)
      if (donate[i]) args[i]->mem.reset();   // the plan's buffer holds it from here on
  // events of a timed execution; destroyed on every exit path unless handed to the executable
  struct EventList {
    std::vector<hipEvent_t> v;
    ~EventList() { for (auto e : v) if (e) (void)hipEventDestroy(e); }
  } evlist;
  std::vector<hipEvent_t>& evs = evlist.v;
  // A timed execution gives every launch its own start and stop event, attached to the dispatch
  // itself (hipExtModuleLaunchKernel): the pair reads the kernel's own begin and end time stamps and
  // puts no marker packets between the kernels.
  const bool timed = launch_ms || profile_async;
  if (timed) {
    evs.assign(2 * P.launches.size(), nullptr);
    for (auto& e : evs) HIP_CHECK(hipEventCreate(&e));
  }
  std::vector<void*> ptrs;
  std::vector<void*> argv;
  for (size_t li = 0; li < P.launches.size(); ++li) {
    const auto& L = P.launches[li];
    ptrs.clear();
    argv.clear();
    for (int b : L.args) {
      if (P.buffers[b].kind == rx::BufferDesc::Fault) { ptrs.push_back(dev->fault_dev); continue; }
      if (!bufs[b]) {
        const auto& B = P.buffers[b];
        if (B.kind == rx::BufferDesc::Param || B.kind == rx::BufferDesc::Const) throw Error("internal: unbound input buffer");
        bufs[b] = std::make_shared<Allocation>(dev, (size_t)B.bytes);
      }
      ptrs.push_back(bufs[b]->ptr);
    }
    for (auto& p : ptrs) argv.push_back(&p);
    // a kernel over an empty tensor has no workgroups: nothing to launch
    const bool empty = L.grid[0] == 0 || L.grid[1] == 0 || L.grid[2] == 0;
    if (timed && !empty) {
      HIP_CHECK(hipExtModuleLaunchKernel(ex->fns[li], L.grid[0] * L.block[0], L.grid[1] * L.block[1], L.grid[2] * L.block[2], L.block[0], L.block[1],
                                         L.block[2], L.lds_bytes, dev->stream, argv.data(), nullptr, evs[2 * li], evs[2 * li + 1], 0));
    } else if (timed) {
      HIP_CHECK(hipEventRecord(evs[2 * li], dev->stream));
      HIP_CHECK(hipEventRecord(evs[2 * li + 1], dev->stream));
    } else if (!empty) {
      HIP_CHECK(hipModuleLaunchKernel(ex->fns[li], L.grid[0], L.grid[1], L.grid[2], L.block[0], L.block[1], L.block[2], L.lds_bytes, dev->stream,
                                      argv.data(), nullptr));
    }
    for (int b : L.args) {
      const auto& B = P.buffers[b];
      if (B.last_use == (int)li && !is_res[b]) bufs[b].reset();
    }
  }
  // result handles and futures made so far; released again if a later step throws
  struct Pending {
    std::vector<RxBuffer*> bufs;
    std::vector<RxFuture*> futs;
    ~Pending() {
      for (RxBuffer* b : bufs) { reg_del(b); delete b; }
      for (RxFuture* f : futs) { if (f->ev) (void)hipEventDestroy(f->ev); delete f; }
    }
  } pending;
  std::vector<RxBuffer*>& new_results = pending.bufs;
  std::vector<RxFuture*>& new_futures = pending.futs;
  for (int r = 0; r < num_results; ++r) {
    const int b = P.result_buffers[r];
    const auto& B = P.buffers[b];
    Mem m = bufs[b];
    if (B.kind == rx::BufferDesc::Const) {
      // a constant returned as a result gets its own copy: the caller may donate it later
      m = std::make_shared<Allocation>(dev, (size_t)B.bytes);
      HIP_CHECK(hipMemcpyAsync(m->ptr, ex->consts[b]->ptr, (size_t)B.bytes, hipMemcpyDeviceToDevice, dev->stream));
    } else if (B.kind == rx::BufferDesc::Param && !m) {
      throw Error("internal: pass-through result lost its storage");
    } else if (B.kind == rx::BufferDesc::Param && !(donate && donate[B.param_index])) {
      // an argument returned unchanged and not donated: the result is a buffer of its own, so that
      // writing into it (CopyToBuffer) or donating it later leaves the caller's argument alone
      m = std::make_shared<Allocation>(dev, std::max<size_t>((size_t)B.bytes, 1));
      if (B.bytes) HIP_CHECK(hipMemcpyAsync(m->ptr, bufs[b]->ptr, (size_t)B.bytes, hipMemcpyDeviceToDevice, dev->stream));
    } else if (!m) {
      m = std::make_shared<Allocation>(dev, (size_t)B.bytes);  // nothing wrote it (empty tensor)
    }
    new_results.push_back(new_buffer(ex->client, dev, P.result_types[r], m));
  }
  if (futures) {
    // A future gets its event when it is first asked (future_event): an event recorded per call costs the stream
    // about 4 us between consecutive executions (0.089 -> 0.0845 ms per call of an 80 us reduction), and all work of a
    // device is ordered on one stream, so an event recorded later completes no earlier than this call's kernels.
    for (int r = 0; r < num_results; ++r) {
      std::unique_ptr<RxFuture> f(new RxFuture);
      f->device = dev;
      new_futures.push_back(f.release());
    }
  }
  if (launch_ms) {
    if (!evs.empty()) HIP_CHECK(hipEventSynchronize(evs.back()));
    for (size_t li = 0; li < P.launches.size(); ++li) HIP_CHECK(hipEventElapsedTime(&launch_ms[li], evs[2 * li], evs[2 * li + 1]));
  }
  // nothing below can fail: publish the results and take the donated arguments' storage
  for (int r = 0; r < num_results; ++r) results[r] = new_results[r];
  new_results.clear();
  if (futures)
    for (int r = 0; r < num_results; ++r) { reg_add(new_futures[r]); futures[r] = new_futures[r]; }
  new_futures.clear();
  donation.committed = true;   // its destructor marks the donated arguments as consumed
  if (profile_async && !launch_ms) {
    ex->pending_events.push_back(std::move(evs));   // read later by RxExecutableTakeTimings
    evs.clear();
  }
}

}  // namespace

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
RX_EXPORT int RxOwns(const void* h) { return h && reg_has(h) ? 1 : 0; }
RX_EXPORT const char* RxLastError(void) { return g_last_error.c_str(); }
RX_EXPORT void RxClearError(void) { g_last_error.clear(); }
RX_EXPORT void InitializeLogs(void) {}
RX_EXPORT void SetLogLevel(int) {}

RX_EXPORT RxClient* MakeGPUClient(int node_id, int num_nodes, int64_t* allowed_devices, int64_t num_allowed_devices, double memory_fraction,
                                  bool preallocate, const char* platform_name, const char** error, void* distributed_runtime_client) {
  (void)preallocate;
  (void)platform_name;
  (void)distributed_runtime_client;
  try {
    if (num_nodes > 1 || node_id != 0) throw Error("INVALID_ARGUMENT: this backend runs one process on one GPU (num_nodes must be 1, node_id 0)");
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) throw Error(std::string("NOT_FOUND: no HIP device is visible (") + hipGetErrorString(e) + ")");
    std::vector<int> ords;
    if (allowed_devices && num_allowed_devices > 0) {
      for (int64_t k = 0; k < num_allowed_devices; ++k) {
        if (allowed_devices[k] < 0 || allowed_devices[k] >= count) throw Error("INVALID_ARGUMENT: allowed device " + std::to_string(allowed_devices[k]) + " does not exist");
        ords.push_back((int)allowed_devices[k]);
      }
    } else ords.push_back(0);
    auto c = std::make_unique<RxClient>();
    for (size_t k = 0; k < ords.size(); ++k) {
      auto d = std::make_unique<RxDevice>();
      d->client = c.get();
      d->ordinal = ords[k];
      d->index = (int)k;
      HIP_CHECK(hipSetDevice(d->ordinal));
      hipDeviceProp_t prop;
      HIP_CHECK(hipGetDeviceProperties(&prop, d->ordinal));
      d->kind = prop.name;
      d->arch = prop.gcnArchName;
      if (d->arch.rfind("gfx950", 0) != 0)
        throw Error("FAILED_PRECONDITION: device " + std::to_string(d->ordinal) + " is " + d->arch + "; this backend only targets gfx950 (MI355X)");
      size_t fr = 0, tot = 0;
      HIP_CHECK(hipMemGetInfo(&fr, &tot));
      d->bytes_limit = (int64_t)((memory_fraction > 0 && memory_fraction <= 1 ? memory_fraction : 1.0) * (double)tot);
      HIP_CHECK(hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking));
      HIP_CHECK(hipGetSymbolAddress(&d->scratch_ptr, HIP_SYMBOL(scratch)));   // with this device current: its own copy
      HIP_CHECK(hipHostMalloc((void**)&d->fault_host, 64, hipHostMallocMapped));
      *d->fault_host = 0;
      HIP_CHECK(hipHostGetDevicePointer(&d->fault_dev, d->fault_host, 0));
      reg_add(d.get());
      c->devices.push_back(std::move(d));
    }
    RxClient* raw = c.release();
    reg_add(raw);
    return raw;
  } catch (const std::exception& ex) {
    g_last_error = ex.what();
    if (error) *error = dup_cstr(ex.what());
    else report_error(ex.what());
    return nullptr;
  }
}

RX_EXPORT void FreeClient(RxClient* c) {
  guarded_void([&] {
    check_client(c);
    c->alive = false;
    for (auto& d : c->devices) {
      (void)hipSetDevice(d->ordinal);
      (void)hipStreamSynchronize(d->stream);
      d->drain(true);
      (void)hipStreamDestroy(d->stream);
      if (d->fault_host) { (void)hipHostFree(d->fault_host); d->fault_host = nullptr; d->fault_dev = nullptr; }
      reg_del(d.get());
    }
    reg_del(c);
    // Buffers freed after this point (late finalizers) still reach their RxDevice through the
    // shared allocation, so the client object itself is kept alive for the life of the process.
  });
}

RX_EXPORT int ClientNumDevices(RxClient* c) { return guarded([&] { check_client(c); return (int)c->devices.size(); }, 0); }
RX_EXPORT int ClientNumAddressableDevices(RxClient* c) { return ClientNumDevices(c); }
RX_EXPORT int ClientProcessIndex(RxClient* c) { return guarded([&] { check_client(c); return 0; }, 0); }
RX_EXPORT RxDevice* ClientGetDevice(RxClient* c, int id) {
  return guarded([&]() -> RxDevice* {
    check_client(c);
    if (id < 0 || id >= (int)c->devices.size()) throw Error("INVALID_ARGUMENT: no device with id " + std::to_string(id));
    return c->devices[id].get();
  }, nullptr);
}
RX_EXPORT RxDevice* ClientGetAddressableDevice(RxClient* c, int id) { return ClientGetDevice(c, id); }
RX_EXPORT const char* ClientGetPlatformName(RxClient* c) {
  return guarded([&]() -> const char* { check_client(c); return dup_cstr("rocm"); }, nullptr);
}
RX_EXPORT void ClientGetDevices(RxClient* c, RxDevice** out) {
  guarded_void([&] { check_client(c); for (size_t k = 0; k < c->devices.size(); ++k) out[k] = c->devices[k].get(); });
}
RX_EXPORT void ClientGetAddressableDevices(RxClient* c, RxDevice** out) { ClientGetDevices(c, out); }
RX_EXPORT const char* DeviceGetKind(RxDevice* d) {
  return guarded([&]() -> const char* { check_device(d); return dup_cstr(d->kind); }, nullptr);
}
RX_EXPORT RxClient* DeviceToClient(RxDevice* d) { return guarded([&]() -> RxClient* { check_device(d); return d->client; }, nullptr); }
RX_EXPORT int64_t PjRtDeviceGetLocalDeviceId(RxDevice* d) { return guarded([&]() -> int64_t { check_device(d); return d->index; }, -1); }
RX_EXPORT int64_t PjRtDeviceGetGlobalDeviceId(RxDevice* d) { return PjRtDeviceGetLocalDeviceId(d); }
RX_EXPORT int64_t PjRtDeviceGetLocalHardwareId(RxDevice* d) { return guarded([&]() -> int64_t { check_device(d); return d->ordinal; }, -1); }
RX_EXPORT bool pjrt_device_is_addressable(RxDevice* d) { return guarded([&] { check_device(d); return true; }, false); }
RX_EXPORT void PjRtDeviceGetAllocatorStats(RxDevice* d, JLAllocatorStats* s) {
  guarded_void([&] {
    check_device(d);
    std::lock_guard<std::mutex> l(d->mu);
    const int64_t none = INT64_MIN;
    s->num_allocs = d->num_allocs;
    s->bytes_in_use = d->bytes_in_use;
    s->peak_bytes_in_use = d->peak_bytes_in_use;
    s->largest_alloc_size = d->largest_alloc;
    s->bytes_limit = d->bytes_limit;
    s->bytes_reserved = 0;
    s->peak_bytes_reserved = 0;
    s->bytes_reservable_limit = none;
    s->largest_free_block_bytes = d->free_blocks.empty() ? 0 : (int64_t)d->free_blocks.rbegin()->first;
    s->pool_bytes = d->pool_bytes;
    s->peak_pool_bytes = d->peak_pool_bytes;
  });
}

RX_EXPORT RxBuffer* ArrayFromHostBuffer(RxClient* c, void* data, uint64_t ptype, size_t dim, const int64_t* cshape, RxDevice* d) {
  return guarded([&]() -> RxBuffer* {
    check_client(c);
    check_device(d);
    rx::TType ty;
    ty.dt = rx::dt_from_code((int)ptype);
    if (ty.dt == rx::DT::INVALID) throw Error("UNIMPLEMENTED: primitive type code " + std::to_string(ptype) + " is not supported");
    for (size_t k = 0; k < dim; ++k) {
      if (cshape[k] < 0) throw Error("INVALID_ARGUMENT: negative dimension");
      ty.dims.push_back(cshape[k]);
    }
    const size_t bytes = (size_t)ty.bytes();
    if (bytes && !data) throw Error("INVALID_ARGUMENT: null host pointer");
    Mem m = std::make_shared<Allocation>(d, std::max<size_t>(bytes, 1));
    if (bytes) {
      HIP_CHECK(hipSetDevice(d->ordinal));
      HIP_CHECK(hipMemcpyAsync(m->ptr, data, bytes, hipMemcpyHostToDevice, d->stream));
      HIP_CHECK(hipStreamSynchronize(d->stream));  // host memory is only borrowed during the call
    }
    return new_buffer(c, d, ty, m);
  }, nullptr);
}

RX_EXPORT RxBuffer* UninitPJRTBuffer(RxClient* c, RxDevice* d, uint64_t ptype, uint64_t shapeLen, uint64_t* shape) {
  return guarded([&]() -> RxBuffer* {
    check_client(c);
    check_device(d);
    rx::TType ty;
    ty.dt = rx::dt_from_code((int)ptype);
    if (ty.dt == rx::DT::INVALID) throw Error("UNIMPLEMENTED: primitive type code " + std::to_string(ptype) + " is not supported");
    for (uint64_t k = 0; k < shapeLen; ++k) ty.dims.push_back((int64_t)shape[k]);
    Mem m = std::make_shared<Allocation>(d, std::max<size_t>((size_t)ty.bytes(), 1));
    return new_buffer(c, d, ty, m);
  }, nullptr);
}

static void live_mem(RxBuffer* b) {
  check_buffer(b);
  if (b->donated || !b->mem) throw Error("INVALID_ARGUMENT: buffer was donated to an execution and can no longer be read");
}

RX_EXPORT void BufferToHost(RxBuffer* b, void* data) {
  guarded_void([&] {
    live_mem(b);
    const size_t bytes = (size_t)b->ty.bytes();
    if (!bytes) return;
    HIP_CHECK(hipSetDevice(b->device->ordinal));
    HIP_CHECK(hipMemcpyAsync(data, b->mem->ptr, bytes, hipMemcpyDeviceToHost, b->device->stream));
    HIP_CHECK(hipStreamSynchronize(b->device->stream));
    check_fault(b->device);
  });
}

RX_EXPORT void CopyToBuffer(RxClient* c, RxBuffer* b, void* data, size_t offset, size_t size, RxBuffer** bufferP) {
  (void)bufferP;
  guarded_void([&] {
    check_client(c);
    live_mem(b);
    if (offset + size > (size_t)b->ty.bytes()) throw Error("INVALID_ARGUMENT: copy range exceeds the buffer");
    HIP_CHECK(hipSetDevice(b->device->ordinal));
    HIP_CHECK(hipMemcpyAsync((char*)b->mem->ptr + offset, data, size, hipMemcpyHostToDevice, b->device->stream));
    HIP_CHECK(hipStreamSynchronize(b->device->stream));
  });
}

RX_EXPORT void CopyFromBuffer(RxClient* c, RxBuffer* b, void* data, size_t offset, size_t size, RxBuffer** bufferP) {
  (void)bufferP;
  guarded_void([&] {
    check_client(c);
    live_mem(b);
    if (offset + size > (size_t)b->ty.bytes()) throw Error("INVALID_ARGUMENT: copy range exceeds the buffer");
    HIP_CHECK(hipSetDevice(b->device->ordinal));
    HIP_CHECK(hipMemcpyAsync(data, (char*)b->mem->ptr + offset, size, hipMemcpyDeviceToHost, b->device->stream));
    HIP_CHECK(hipStreamSynchronize(b->device->stream));
    check_fault(b->device);
  });
}

RX_EXPORT const int64_t* BufferShape(RxBuffer* b) { return guarded([&]() -> const int64_t* { check_buffer(b); return b->ty.dims.data(); }, nullptr); }
RX_EXPORT int64_t BufferNDimensions(RxBuffer* b) { return guarded([&]() -> int64_t { check_buffer(b); return (int64_t)b->ty.dims.size(); }, 0); }
RX_EXPORT int BufferPrimitiveType(RxBuffer* b) { return guarded([&] { check_buffer(b); return rx::info(b->ty.dt).code; }, 0); }
RX_EXPORT RxDevice* BufferToDevice(RxBuffer* b) { return guarded([&]() -> RxDevice* { check_buffer(b); return b->device; }, nullptr); }
RX_EXPORT RxClient* BufferToClient(RxBuffer* b) { return guarded([&]() -> RxClient* { check_buffer(b); return b->client; }, nullptr); }
RX_EXPORT uint8_t BufferOnCPU(RxBuffer* b) { return guarded([&]() -> uint8_t { check_buffer(b); return 0; }, 0); }
RX_EXPORT void* UnsafeBufferPointer(RxBuffer* b) { return guarded([&]() -> void* { live_mem(b); return b->mem->ptr; }, nullptr); }
RX_EXPORT RxBuffer* CopyBufferToDevice(RxBuffer* b, RxDevice* dst) {
  return guarded([&]() -> RxBuffer* {
    live_mem(b);
    check_device(dst);
    const size_t bytes = (size_t)b->ty.bytes();
    Mem m = std::make_shared<Allocation>(dst, std::max<size_t>(bytes, 1));
    if (bytes) {
      HIP_CHECK(hipSetDevice(dst->ordinal));
      HIP_CHECK(hipMemcpyAsync(m->ptr, b->mem->ptr, bytes, hipMemcpyDeviceToDevice, dst->stream));
      if (dst != b->device) HIP_CHECK(hipStreamSynchronize(dst->stream));
    }
    return new_buffer(dst->client, dst, b->ty, m);
  }, nullptr);
}
RX_EXPORT void PjRtBufferFree(RxBuffer* b) {
  // called from finalizers: tolerate null and handles that are already gone
  if (!b || !reg_has(b)) return;
  reg_del(b);
  delete b;
}

RX_EXPORT int RxCompileOffline(const char* text, size_t len, int with_source, char** report) {
  try {
    rx::Graph g = rx::parse_module(text, len);
    rx::Plan p = rx::make_plan(g, plan_options());
    std::string code = rtc_compile(p.source, "gfx950");
    if (report) {
      std::string r = p.report() + "code object: " + std::to_string(code.size()) + " bytes\n";
      if (with_source) r += "----- source -----\n" + p.source;
      *report = dup_cstr(r);
    }
    return 0;
  } catch (const std::exception& e) {
    g_last_error = e.what();
    if (report) *report = dup_cstr(e.what());
    return 1;
  }
}

namespace {
// Parse, plan and load the module text of an executable: kernels through hiprtc, constants to the device.
void load_plan(RxExecutable* ex, rx::PlanOptions opt) {
  RxDevice* d = ex->device;
  if (d->waits_failed) opt.single_pass_scan = false;   // a wait between workgroups has expired on this device before
  try {
    rx::Graph g = rx::parse_module(ex->text.data(), ex->text.size());
    ex->plan = rx::make_plan(g, opt);
  } catch (const std::exception& e) {
    // same shape of message as the reference: module text followed by the status (API.cpp:1499-1505)
    throw Error(ex->text.substr(0, 4000) + "\n" + e.what());
  }
  ex->report = ex->plan.report();
  ex->waits = false;
  for (auto& B : ex->plan.buffers) ex->waits = ex->waits || B.kind == rx::BufferDesc::Fault;
  HIP_CHECK(hipSetDevice(d->ordinal));
  ex->fns.clear();
  if (!ex->plan.launches.empty()) {
    std::string code = rtc_compile(ex->plan.source, d->arch);
    HIP_CHECK(hipModuleLoadData(&ex->module, code.data()));
    for (auto& L : ex->plan.launches) {
      hipFunction_t f;
      HIP_CHECK(hipModuleGetFunction(&f, ex->module, L.kernel.c_str()));
      if (L.lds_bytes > 48 * 1024) {
        // more dynamic LDS than the default limit: gfx950 has 160 KB per workgroup
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(f), hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.lds_bytes);
        if (e != hipSuccess) {
          (void)hipGetLastError();
          throw Error("kernel " + L.kernel + " needs " + std::to_string(L.lds_bytes) + " bytes of LDS, which the device refused (" +
                      hipGetErrorString(e) + ")");
        }
      }
      ex->fns.push_back(f);
    }
  }
  ex->consts.assign(ex->plan.buffers.size(), Mem());
  for (size_t b = 0; b < ex->plan.buffers.size(); ++b) {
    auto& B = ex->plan.buffers[b];
    if (B.kind != rx::BufferDesc::Const) continue;
    ex->consts[b] = std::make_shared<Allocation>(d, std::max<size_t>(B.data.size(), 1));
    // on the device's stream: the block may have been recycled from a buffer whose last kernel
    // is still queued there, and a copy on the null stream would not wait for it
    if (!B.data.empty()) HIP_CHECK(hipMemcpyAsync(ex->consts[b]->ptr, B.data.data(), B.data.size(), hipMemcpyHostToDevice, d->stream));
  }
  HIP_CHECK(hipStreamSynchronize(d->stream));   // pageable host data: wait before the plan may move
}

// After a wait between workgroups has expired on the device (check_fault), an executable whose kernels wait is rebuilt
// from its module text in the form that does not wait (two launches per scan).  Called with ex->mu held.
void rebuild_without_waits(RxExecutable* ex) {
  if (!ex->waits || !ex->device->waits_failed) return;
  HIP_CHECK(hipSetDevice(ex->device->ordinal));
  HIP_CHECK(hipStreamSynchronize(ex->device->stream));   // kernels of the old module may still be queued
  if (ex->module) { (void)hipModuleUnload(ex->module); ex->module = nullptr; }
  for (auto& evs : ex->pending_events)   // timings of the old plan's launches
    for (auto& e : evs) (void)hipEventDestroy(e);
  ex->pending_events.clear();
  load_plan(ex, plan_options());
}
}  // namespace

RX_EXPORT RxExecutable* ClientCompileFromText(RxClient* c, const char* text, size_t len, const char* opts, size_t nopts) {
  (void)opts;
  (void)nopts;
  return guarded([&]() -> RxExecutable* {
    check_client(c);
    if (!text) throw Error("INVALID_ARGUMENT: null module text");
    RxDevice* d = c->devices[0].get();
    std::unique_ptr<RxExecutable> ex(new RxExecutable);
    ex->client = c;
    ex->device = d;
    ex->text.assign(text, len);
    load_plan(ex.get(), plan_options());
    RxExecutable* raw = ex.release();
    reg_add(raw);
    return raw;
  }, nullptr);
}

RX_EXPORT void ExecutableFree(RxExecutable* ex) {
  if (!ex || !reg_has(ex)) return;
  reg_del(ex);
  if (ex->module) {
    (void)hipSetDevice(ex->device->ordinal);
    (void)hipStreamSynchronize(ex->device->stream);
    (void)hipModuleUnload(ex->module);
  }
  for (auto& evs : ex->pending_events)
    for (auto& e : evs) (void)hipEventDestroy(e);
  delete ex;
}
RX_EXPORT RxClient* PjRtLoadedExecutableGetClient(RxExecutable* ex) { return guarded([&]() -> RxClient* { check_exec(ex); return ex->client; }, nullptr); }
RX_EXPORT void PjRtLoadedExecutableGetHloModules(RxExecutable* ex, void** mods, int32_t* n) {
  (void)mods;
  guarded_void([&] { check_exec(ex); if (n) *n = 0; });
}
// The counterpart of pjrt_hlo_module_cost_analysis_properties (API.cpp:3238-3260) for an executable of this library,
// which keeps no HLO module: the same eleven floats, counted over the StableHLO module as it was compiled.  The optimal
// time is that of the plan's launches at the device's peaks (each launch the larger of its arithmetic and its memory time).
RX_EXPORT void RxExecutableCostAnalysis(RxExecutable* ex, float* props11) {
  guarded_void([&] {
    check_exec(ex);
    if (!props11) throw Error("INVALID_ARGUMENT: null properties");
    std::lock_guard<std::mutex> lock(ex->mu);
    const rx::Plan& P = ex->plan;
    double optimal = 0;
    for (auto& L : P.launches) {
      const double peak = L.kind == "gemm_f8" ? 5.0e15 : (L.kind == "gemm_bf16" || L.kind == "gemm_f16" || L.kind == "conv_bf16" || L.kind == "conv_f16") ? 2.5e15 : L.kind == "gemm_f64" ? 78.6e12 : 157.3e12;
      optimal += std::max(L.flops / peak, L.algo_bytes / 8.0e12);
    }
    const double mem_time = P.hlo_bytes_accessed / 8.0e12;
    props11[0] = (float)P.hlo_flops;
    props11[1] = (float)P.hlo_transcendentals;
    props11[2] = (float)P.hlo_bytes_accessed;
    props11[3] = (float)optimal;
    props11[4] = (float)(mem_time > 0 ? std::min(1.0, optimal / mem_time) : 0.0);   // utilization: optimal time over the time of every op's own traffic
    props11[5] = P.hlo_bytes_accessed > 0 ? (float)(P.hlo_operand_bytes[0] / P.hlo_bytes_accessed) : 0.f;
    props11[6] = P.hlo_bytes_accessed > 0 ? (float)(P.hlo_operand_bytes[1] / P.hlo_bytes_accessed) : 0.f;
    props11[7] = (float)P.hlo_operand_bytes[0];
    props11[8] = (float)P.hlo_operand_bytes[1];
    props11[9] = (float)P.hlo_output_bytes;
    props11[10] = 0.f;
  });
}
RX_EXPORT const char* RxExecutableReport(RxExecutable* ex) { return guarded([&]() -> const char* { check_exec(ex); return ex->report.c_str(); }, ""); }
RX_EXPORT int RxExecutableNumLaunches(RxExecutable* ex) { return guarded([&] { check_exec(ex); return (int)ex->plan.launches.size(); }, 0); }
RX_EXPORT int RxExecutableNumResults(RxExecutable* ex) { return guarded([&] { check_exec(ex); return (int)ex->plan.result_types.size(); }, 0); }
RX_EXPORT void RxExecutableLaunchInfo(RxExecutable* ex, int i, const char** kernel, const char** kind, double* bytes, double* flops) {
  guarded_void([&] {
    check_exec(ex);
    if (i < 0 || i >= (int)ex->plan.launches.size()) throw Error("INVALID_ARGUMENT: launch index out of range");
    auto& L = ex->plan.launches[i];
    if (kernel) *kernel = L.kernel.c_str();
    if (kind) *kind = L.kind.c_str();
    if (bytes) *bytes = L.algo_bytes;
    if (flops) *flops = L.flops;
  });
}

RX_EXPORT void XLAExecuteSharded(RxExecutable* ex, int num_args, RxBuffer** op_args, RxDevice* device, uint8_t* is_arg_donatable, int num_results,
                                 RxBuffer** op_results, uint8_t* futures, RxFuture** future_results) {
  guarded_void([&] {
    if (futures) *futures = future_results ? 1 : 0;
    execute(ex, num_args, op_args, device, is_arg_donatable, num_results, op_results, nullptr, future_results);
  });
}
RX_EXPORT void RxExecuteTimed(RxExecutable* ex, int num_args, RxBuffer** op_args, RxDevice* device, uint8_t* is_arg_donatable, int num_results,
                              RxBuffer** op_results, float* launch_ms) {
  guarded_void([&] { execute(ex, num_args, op_args, device, is_arg_donatable, num_results, op_results, launch_ms, nullptr); });
}

RX_EXPORT void RxExecuteProfiled(RxExecutable* ex, int num_args, RxBuffer** op_args, RxDevice* device, uint8_t* is_arg_donatable, int num_results,
                                 RxBuffer** op_results) {
  guarded_void([&] { execute(ex, num_args, op_args, device, is_arg_donatable, num_results, op_results, nullptr, nullptr, true); });
}
RX_EXPORT int RxExecutableTakeTimings(RxExecutable* ex, double* launch_ms_sum) {
  return guarded([&]() -> int {
    check_exec(ex);
    std::lock_guard<std::mutex> lock(ex->mu);
    const size_t nl = ex->plan.launches.size();
    for (size_t li = 0; li < nl; ++li) launch_ms_sum[li] = 0.0;
    int runs = 0;
    HIP_CHECK(hipSetDevice(ex->device->ordinal));
    for (auto& evs : ex->pending_events) {
      if (!evs.empty()) HIP_CHECK(hipEventSynchronize(evs.back()));
      for (size_t li = 0; li < nl; ++li) {
        float ms = 0.f;
        HIP_CHECK(hipEventElapsedTime(&ms, evs[2 * li], evs[2 * li + 1]));
        launch_ms_sum[li] += ms;
      }
      for (auto& e : evs) (void)hipEventDestroy(e);
      ++runs;
    }
    ex->pending_events.clear();
    return runs;
  }, 0);
}

// The launch list of `ex` with caller-owned results and every temporary inside the device's static
// scratch array: no allocation, no event, no handle is created.
RX_EXPORT int RxExecuteNoAlloc(RxExecutable* ex, int num_args, RxBuffer** args, int num_results, RxBuffer** results) {
  return guarded([&]() -> int {
    check_exec(ex);
    RxDevice* dev = ex->device;
    std::lock_guard<std::mutex> lock(ex->mu);
    if (ex->waits && dev->waits_failed)
      throw Error("FAILED_PRECONDITION: a wait between workgroups expired on this device earlier; this executable has to be rebuilt in the form "
                  "that does not wait, which allocates: execute it once through XLAExecuteSharded");
    const rx::Plan& P = ex->plan;
    if (num_args != (int)P.param_types.size())
      throw Error("INVALID_ARGUMENT: executable expects " + std::to_string(P.param_types.size()) + " arguments, got " + std::to_string(num_args));
    if (num_results != (int)P.result_types.size())
      throw Error("INVALID_ARGUMENT: executable returns " + std::to_string(P.result_types.size()) + " results, got room for " + std::to_string(num_results));
    for (int i = 0; i < num_args; ++i) {
      check_buffer(args[i]);
      if (args[i]->donated || !args[i]->mem) throw Error("INVALID_ARGUMENT: argument " + std::to_string(i) + " was donated to an earlier execution");
      if (!(args[i]->ty == P.param_types[i]))
        throw Error("INVALID_ARGUMENT: argument " + std::to_string(i) + " has type " + args[i]->ty.str() + ", executable expects " + P.param_types[i].str());
      if (args[i]->device != dev) throw Error("INVALID_ARGUMENT: argument " + std::to_string(i) + " lives on another device");
    }
    for (int r = 0; r < num_results; ++r) {
      check_buffer(results[r]);
      if (results[r]->donated || !results[r]->mem) throw Error("INVALID_ARGUMENT: result buffer " + std::to_string(r) + " was donated to an earlier execution");
      if (!(results[r]->ty == P.result_types[r]))
        throw Error("INVALID_ARGUMENT: result buffer " + std::to_string(r) + " has type " + results[r]->ty.str() + ", executable returns " + P.result_types[r].str());
      if (results[r]->device != dev) throw Error("INVALID_ARGUMENT: result buffer " + std::to_string(r) + " lives on another device");
      for (int i = 0; i < num_args; ++i)
        if (args[i]->mem->ptr == results[r]->mem->ptr) throw Error("INVALID_ARGUMENT: result buffer " + std::to_string(r) + " is also argument " + std::to_string(i));
      for (int q = 0; q < r; ++q)
        if (results[q]->mem->ptr == results[r]->mem->ptr) throw Error("INVALID_ARGUMENT: result buffers " + std::to_string(q) + " and " + std::to_string(r) + " are the same");
    }
    if (!dev->scratch_ptr) throw Error("internal: the device's scratch array was not resolved");
    // where every plan buffer lives: arguments, constants of the executable, the caller's results
    // (first result that returns the buffer), everything else at 256-byte steps in the scratch array
    const size_t NB = P.buffers.size();
    std::vector<void*> where(NB, nullptr);
    std::vector<int> first_result(NB, -1);
    for (int r = 0; r < num_results; ++r)
      if (first_result[P.result_buffers[r]] < 0) first_result[P.result_buffers[r]] = r;
    size_t used = 0;
    for (size_t b = 0; b < NB; ++b) {
      const auto& B = P.buffers[b];
      if (B.kind == rx::BufferDesc::Param) where[b] = args[B.param_index]->mem->ptr;
      else if (B.kind == rx::BufferDesc::Const) where[b] = ex->consts[b]->ptr;
      else if (B.kind == rx::BufferDesc::Fault) where[b] = dev->fault_dev;
      else if (first_result[b] >= 0) where[b] = results[first_result[b]]->mem->ptr;
      else if (B.first_def >= 0 || B.last_use >= 0) {
        where[b] = (char*)dev->scratch_ptr + used;
        used += ((size_t)B.bytes + 255) & ~(size_t)255;
      }
    }
    if (used > RX_NOALLOC_SCRATCH_BYTES)
      throw Error("RESOURCE_EXHAUSTED: the temporaries of this executable take " + std::to_string(used) + " bytes; RxExecuteNoAlloc holds at most " +
                  std::to_string(RX_NOALLOC_SCRATCH_BYTES) + " (use XLAExecuteSharded)");
    std::lock_guard<std::mutex> slock(dev->scratch_mu);
    HIP_CHECK(hipSetDevice(dev->ordinal));
    std::vector<void*> ptrs, argv;
    for (size_t li = 0; li < P.launches.size(); ++li) {
      const auto& L = P.launches[li];
      if (L.grid[0] == 0 || L.grid[1] == 0 || L.grid[2] == 0) continue;
      ptrs.clear();
      argv.clear();
      for (int b : L.args) {
        if (!where[b]) throw Error("internal: unbound buffer in launch " + std::to_string(li));
        ptrs.push_back(where[b]);
      }
      for (auto& p : ptrs) argv.push_back(&p);
      HIP_CHECK(hipModuleLaunchKernel(ex->fns[li], L.grid[0], L.grid[1], L.grid[2], L.block[0], L.block[1], L.block[2], L.lds_bytes, dev->stream,
                                      argv.data(), nullptr));
    }
    // results that no kernel of this call wrote in place: arguments and constants returned as they
    // are, and a buffer returned more than once
    for (int r = 0; r < num_results; ++r) {
      const int b = P.result_buffers[r];
      const auto& B = P.buffers[b];
      void* src = where[b];
      if (src && src != results[r]->mem->ptr && B.bytes && P.result_types[r].bytes())
        HIP_CHECK(hipMemcpyAsync(results[r]->mem->ptr, src, (size_t)P.result_types[r].bytes(), hipMemcpyDeviceToDevice, dev->stream));
    }
    return 0;
  }, 1);
}
RX_EXPORT size_t RxNoAllocScratchBytes(void) { return RX_NOALLOC_SCRATCH_BYTES; }

RX_EXPORT void FreeFuture(RxFuture* f) {
  if (!f || !reg_has(f)) return;
  reg_del(f);
  if (f->ev) (void)hipEventDestroy(f->ev);
  delete f;
}
// The event of a future, recorded on its device's stream the first time the future is asked about.
static void future_event(RxFuture* f) {
  std::lock_guard<std::mutex> l(f->device->future_mu);   // two threads may ask the same future at once
  if (f->ev || f->done) return;
  if (!f->device->client || !f->device->client->alive.load()) { f->done = true; return; }   // FreeClient drained the stream
  HIP_CHECK(hipSetDevice(f->device->ordinal));
  HIP_CHECK(hipEventCreateWithFlags(&f->ev, hipEventDisableTiming));
  HIP_CHECK(hipEventRecord(f->ev, f->device->stream));
}
RX_EXPORT uint8_t FutureIsReady(RxFuture* f) {
  return guarded([&]() -> uint8_t {
    if (!f || !reg_has(f)) throw Error("INVALID_ARGUMENT: null or foreign future handle");
    future_event(f);
    if (f->done) return 1;
    hipError_t e = hipEventQuery(f->ev);
    if (e == hipSuccess) { check_fault(f->device); return 1; }
    if (e == hipErrorNotReady) { (void)hipGetLastError(); return 0; }
    throw Error(std::string("execution failed: ") + hipGetErrorString(e));
  }, 0);
}
RX_EXPORT void FutureAwait(RxFuture* f) {
  guarded_void([&] {
    if (!f || !reg_has(f)) throw Error("INVALID_ARGUMENT: null or foreign future handle");
    future_event(f);
    if (f->done) return;
    hipError_t e = hipEventSynchronize(f->ev);
    if (e != hipSuccess) throw Error(std::string("execution failed: ") + hipGetErrorString(e));
    check_fault(f->device);
  });
}
RX_EXPORT void RxDeviceSynchronize(RxDevice* d) {
  guarded_void([&] { check_device(d); HIP_CHECK(hipSetDevice(d->ordinal)); HIP_CHECK(hipStreamSynchronize(d->stream)); check_fault(d); });
}

RX_EXPORT int RxMfmaCeiling(RxDevice* d, int kind, int zero_operands, double* tflops, double* clock_mhz) {
  return guarded([&]() -> int {
    check_device(d);
    if (kind != 0 && kind != 1) throw Error("INVALID_ARGUMENT: kind is 0 (bf16) or 1 (f8E4M3FN)");
    HIP_CHECK(hipSetDevice(d->ordinal));
    Allocation ticks(d, (2 * 1024 + 8) * sizeof(unsigned long long));
    HIP_CHECK(hipMemsetAsync(ticks.ptr, 0, (2 * 1024 + 8) * sizeof(unsigned long long), d->stream));
    // 256 workgroups of four wavefronts: one wavefront per SIMD of the chip.  About 10 ms per launch, so that the
    // clock has settled under the power limit; the second launch is the one that is timed.
    const int iters = 40000;
    const double flop_per_iter = kind == 0 ? 32 * 2.0 * 16 * 16 * 32 : 16 * 2.0 * 16 * 16 * 128;
    hipEvent_t a, b;
    HIP_CHECK(hipEventCreate(&a));
    HIP_CHECK(hipEventCreate(&b));
    auto launch = [&]() {
      if (kind == 0) hipLaunchKernelGGL(rx_mfma_probe<0>, dim3(256), dim3(256), 0, d->stream, (unsigned long long*)ticks.ptr, iters, zero_operands);
      else hipLaunchKernelGGL(rx_mfma_probe<1>, dim3(256), dim3(256), 0, d->stream, (unsigned long long*)ticks.ptr, iters, zero_operands);
    };
    launch();
    HIP_CHECK(hipEventRecord(a, d->stream));
    launch();
    HIP_CHECK(hipEventRecord(b, d->stream));
    HIP_CHECK(hipEventSynchronize(b));
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    std::vector<unsigned long long> h(2 * 1024);
    HIP_CHECK(hipMemcpy(h.data(), ticks.ptr, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    double c = 0, w = 0;
    for (int i = 0; i < 1024; ++i) { c += (double)h[2 * i]; w += (double)h[2 * i + 1]; }
    if (tflops) *tflops = flop_per_iter * iters * 1024 / (ms * 1e-3) / 1e12;
    if (clock_mhz) *clock_mhz = w > 0 ? c / w * 100.0 : 0.0;   // the real-time counter ticks at 100 MHz
    return 0;
  }, 1);
}

RX_EXPORT int RxGemmClockProbe(RxDevice* d, int kind, double* out8) {
  return guarded([&]() -> int {
    check_device(d);
    if (kind < 0 || kind > 2) throw Error("INVALID_ARGUMENT: kind is 0 (bf16 8192 x 4096 x 4096), 1 (f8E4M3FN 8192^3) or 2 (the bf16 product on the ping-pong body)");
    if (!out8) throw Error("INVALID_ARGUMENT: null result array");
    HIP_CHECK(hipSetDevice(d->ordinal));
    const size_t M = 8192, N = kind == 1 ? 8192 : 4096, K = kind == 1 ? 8192 : 4096, esz = kind == 1 ? 1 : 2;
    const unsigned grid = (unsigned)rx::gemm_grid((int64_t)(M / 256), (int64_t)(N / 256), 4, 8);
    Allocation a(d, M * K * esz), b(d, N * K * esz), o(d, M * N * 2), sl(d, grid * 48), lf(d, grid * 16);
    hipLaunchKernelGGL(rx_probe_fill, dim3(4096), dim3(256), 0, d->stream, a.ptr, M * K, kind == 1 ? 2 : 0, 1u);
    hipLaunchKernelGGL(rx_probe_fill, dim3(4096), dim3(256), 0, d->stream, b.ptr, N * K, kind == 1 ? 2 : 1, 77u);
    HIP_CHECK(hipMemsetAsync(sl.ptr, 0, grid * 48, d->stream));
    HIP_CHECK(hipMemsetAsync(lf.ptr, 0, grid * 16, d->stream));
    const int lds = 2 * 512 * 128;
    auto fn = kind == 0 ? rx_gemm_clock_probe<0> : (kind == 1 ? rx_gemm_clock_probe<1> : rx_gemm_clock_probe<2>);
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    // Back to back, and not timed before the device has been under this load for 150 ms: after an idle period the first
    // 20 ms or so of a load run up to 20 % slower (8192 x 4096 x 4096 bf16: 246 us per launch 5 ms after the start,
    // 201 us from 22 ms on), whatever the kernel.
    const int reps = 20;
    // RX_PROBE_SETTLE_MS: that time (counter runs, which record every dispatch, set it to 0)
    const float settle_ms = getenv("RX_PROBE_SETTLE_MS") ? (float)atof(getenv("RX_PROBE_SETTLE_MS")) : 150.f;
    HIP_CHECK(hipEventRecord(e0, d->stream));
    for (;;) {
      for (int i = 0; i < 20; ++i) hipLaunchKernelGGL(fn, dim3(grid), dim3(512), lds, d->stream, a.ptr, b.ptr, (rx_u16*)o.ptr, (unsigned long long*)sl.ptr, (unsigned long long*)lf.ptr);
      HIP_CHECK(hipEventRecord(e1, d->stream));
      HIP_CHECK(hipEventSynchronize(e1));
      float warm_ms = 0;
      HIP_CHECK(hipEventElapsedTime(&warm_ms, e0, e1));
      if (warm_ms >= settle_ms) break;
    }
    HIP_CHECK(hipEventRecord(e0, d->stream));
    for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(fn, dim3(grid), dim3(512), lds, d->stream, a.ptr, b.ptr, (rx_u16*)o.ptr, (unsigned long long*)sl.ptr, (unsigned long long*)lf.ptr);
    HIP_CHECK(hipEventRecord(e1, d->stream));
    HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    std::vector<unsigned long long> hs(grid * 6), hl(grid * 2);
    HIP_CHECK(hipMemcpy(hs.data(), sl.ptr, grid * 48, hipMemcpyDeviceToHost));
    HIP_CHECK(hipMemcpy(hl.data(), lf.ptr, grid * 16, hipMemcpyDeviceToHost));
    double sc = 0, sr = 0, lc = 0, lr = 0;
    int ns = 0;
    double pc = 0, pr = 0, pn = 0;
    for (unsigned w = 0; w < grid; ++w) {
      if (kind == 2) { for (int g = 0; g < 2; ++g) { pc += (double)hs[(2 * w + g) * 3]; pr += (double)hs[(2 * w + g) * 3 + 1]; pn += (double)hs[(2 * w + g) * 3 + 2]; } }
      else if (hs[2 * w + 1]) { sc += (double)hs[2 * w]; sr += (double)hs[2 * w + 1]; ++ns; }
      lc += (double)hl[2 * w]; lr += (double)hl[2 * w + 1];
    }
    const double us = ms * 1e3 / reps;
    out8[0] = us;                                                   // per launch; the sleeping wavefronts lengthen it by a few per cent
    out8[1] = 2.0 * M * N * K / (us * 1e-6) / 1e12;                 // TFLOP/s
    out8[2] = lr > 0 ? lc / lr * 100.0 : 0.0;                       // cycle counter / real time over the workgroups' lifetimes, MHz
    out8[3] = sr > 0 ? sc / sr * 100.0 : 0.0;                       // the same over the sleeps, MHz (kinds 0 and 1)
    out8[4] = ns > 0 ? sc / ns : 0.0;                               // cycles counted over a sleep of 65024 nominal cycles
    out8[5] = pn > 0 ? pc / pn : 0.0;                               // kind 2: cycles per compute phase of 64 MFMAs issued back to back
    out8[6] = pr > 0 ? pc / pr * 100.0 : 0.0;                       // kind 2: cycle counter / real time over those phases, MHz
    out8[7] = pn > 0 ? pr / pn * 10.0 : 0.0;                        // kind 2: nanoseconds per compute phase
    return 0;
  }, 1);
}

RX_EXPORT float RxCalibrationCopy(RxDevice* d, size_t bytes, int iters) {
  return guarded([&]() -> float {
    check_device(d);
    if (iters < 1) iters = 1;
    bytes &= ~(size_t)15;
    if (!bytes) throw Error("INVALID_ARGUMENT: copy size must be at least 16 bytes");
    HIP_CHECK(hipSetDevice(d->ordinal));
    Allocation src(d, bytes), dst(d, bytes);
    HIP_CHECK(hipMemsetAsync(src.ptr, 1, bytes, d->stream));
    const size_t n16 = bytes / 16;
    // one 16-byte element per thread, workgroups in address order: 6.2-6.5 TB/s of read + write on this part; a
    // grid-stride loop over 8192 workgroups, whose accesses drift apart, reaches 4.6
    const unsigned grid = (unsigned)std::min<size_t>((n16 + 255) / 256, 0x7fffffffu);
    hipEvent_t a, b;
    HIP_CHECK(hipEventCreate(&a));
    HIP_CHECK(hipEventCreate(&b));
    hipLaunchKernelGGL(rx_copy16, dim3(grid), dim3(256), 0, d->stream, (const uint4*)src.ptr, (uint4*)dst.ptr, n16);  // warm-up
    HIP_CHECK(hipEventRecord(a, d->stream));
    for (int i = 0; i < iters; ++i) hipLaunchKernelGGL(rx_copy16, dim3(grid), dim3(256), 0, d->stream, (const uint4*)src.ptr, (uint4*)dst.ptr, n16);
    HIP_CHECK(hipEventRecord(b, d->stream));
    HIP_CHECK(hipEventSynchronize(b));
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    return ms / (float)iters;
  }, -1.0f);
}
