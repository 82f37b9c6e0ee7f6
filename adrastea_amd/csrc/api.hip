// extern "C" entry points: argument validation, kernel selection, launch.
// Declarations and the reference interface each one replaces: include/adrastea_kernels.h.
#include <string.h>

#include <atomic>
#include <mutex>

#include "adr_common.hpp"

using namespace adr;

namespace adr {
int set_knob(int id, int value);  // device.hip
}

namespace {

constexpr int ABI_VERSION = 1;

int validate_matmul(const MatmulArgs& a, bool check_ptrs) {
  if (a.store > ADR_STORE_QUICK_GELU_BIAS || a.load > ADR_LOAD_SCALE || a.mask > ADR_MASK_CAUSAL)
    return ADR_EINVAL_ENUM;
  if (a.store == ADR_STORE_GELU_BIAS) return ADR_ENOTIMPL;
  if (a.batches < 0 || a.m < 0 || a.n < 0 || a.k < 0) return ADR_EINVAL_SHAPE;
  // Element offsets are 32-bit integers in the reference (every kernel argument is an i32,
  // kernels.rs:864-887, and its kernels index with int): a view whose farthest element lies at or
  // beyond 2^31 elements cannot be addressed there, and is rejected here rather than wrapped.
  if (a.batches && a.m && a.n) {
    auto span = [](int64_t d0, int64_t s0, int64_t d1, int64_t s1, int64_t d2, int64_t s2) {
      auto mag = [](int64_t v) { return v < 0 ? -v : v; };
      return (d0 ? (d0 - 1) * mag(s0) : 0) + (d1 ? (d1 - 1) * mag(s1) : 0) +
             (d2 ? (d2 - 1) * mag(s2) : 0);
    };
    const int64_t lim = (int64_t)1 << 31;
    if (span(a.n, a.stride_ox, a.m, a.stride_oy, a.batches, a.stride_oz) >= lim ||
        span(a.k, a.stride_lx, a.m, a.stride_ly, a.batches, a.stride_lz) >= lim ||
        span(a.n, a.stride_rx, a.k, a.stride_ry, a.batches, a.stride_rz) >= lim)
      return ADR_EINVAL_SHAPE;
  }
  if (check_ptrs) {
    if (a.batches && a.m && a.n) {
      if (!a.output || (a.k && (!a.lhs || !a.rhs))) return ADR_ENULL;
      if (Epilogue::needs_bias(a.store) && !a.bias) return ADR_ENULL;
    }
  }
  return ADR_OK;
}

MatmulArgs pack(uint16_t* output, const uint16_t* lhs, const uint16_t* rhs, int32_t batches,
                int32_t m, int32_t k, int32_t n, int32_t stride_ox, int32_t stride_oy,
                int32_t stride_oz, int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                int32_t stride_rx, int32_t stride_ry, int32_t stride_rz, const uint16_t* bias,
                float beta, float scale, uint32_t store, uint32_t load, uint32_t mask) {
  MatmulArgs a{};
  a.output = (half_t*)output;
  a.lhs = (const half_t*)lhs;
  a.rhs = (const half_t*)rhs;
  a.batches = batches; a.m = m; a.k = k; a.n = n;
  a.stride_ox = stride_ox; a.stride_oy = stride_oy; a.stride_oz = stride_oz;
  a.stride_lx = stride_lx; a.stride_ly = stride_ly; a.stride_lz = stride_lz;
  a.stride_rx = stride_rx; a.stride_ry = stride_ry; a.stride_rz = stride_rz;
  a.bias = (const half_t*)bias;
  a.beta = beta;
  a.scale = scale;
  a.store = store; a.load = load; a.mask = mask;
  return a;
}

bool empty(const MatmulArgs& a) { return a.batches == 0 || a.m == 0 || a.n == 0; }

// Every launching entry point starts here: ADR_EUNSUPPORTED_DEVICE unless the current device is
// a gfx950 (the kernels are built for nothing else), or the error of the failed device query.
int check_device() { return device_info().status; }

int run_matmul(hipStream_t stream, const MatmulArgs& a, bool allow_fast) {
  if (empty(a)) return ADR_OK;
  if (int rc = check_device()) return rc;
  const char* name;
  if (allow_fast && gemv_f16_supported(a, &name)) return (int)launch_gemv_f16(stream, a);
  if (allow_fast && mfma_gemm_supported(a, &name)) return (int)launch_mfma_gemm(stream, a);
  return (int)launch_matmul_general(stream, a);  // also the k == 0 case: store(0)
}

adr_tensor_desc desc2d(const void* ptr, int rows, int cols) {
  adr_tensor_desc d{};
  d.ptr = (void*)ptr;
  d.dims = 2;
  d.shape[0] = (uint32_t)cols; d.shape[1] = (uint32_t)rows;
  d.strides[0] = 1; d.strides[1] = (uint32_t)cols;
  return d;
}

int validate_quant(const adr_tensor_desc& wide, const adr_tensor_desc& scales,
                   const adr_tensor_desc& other) {
  if (!wide.ptr || !scales.ptr || !other.ptr) return ADR_ENULL;
  if (wide.dims != 2 || scales.dims != 2 || other.dims != 2) return ADR_EINVAL_SHAPE;
  if (wide.shape[0] != other.shape[0] || wide.shape[1] != other.shape[1] ||
      scales.shape[1] != wide.shape[1])
    return ADR_EINVAL_SHAPE;
  if (scales.shape[0] == 0 || wide.shape[0] % scales.shape[0] != 0) return ADR_EDIVISIBILITY;
  return ADR_OK;
}

}  // namespace

// ---- scratch of the entry point that allocates nothing ------------------------------------------
// A file-scope device array: every GPU the library runs on holds its own copy, at its own
// address, until the process ends.  In host code the array's NAME is only a handle for
// hipGetSymbolAddress: the kernels get the device address that call returns, kept per device.
static __device__ __align__(256) unsigned char scratch[ADR_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int MAX_SCRATCH_DEVICES = 64;
std::atomic<void*> scratch_address[MAX_SCRATCH_DEVICES];

// Device address of `scratch` on the current device (looked up once per device, with that device
// current), or null with the error in *err.
void* scratch_on_current_device(hipError_t* err) {
  *err = hipSuccess;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_SCRATCH_DEVICES) {
    *err = e != hipSuccess ? e : hipErrorInvalidDevice;
    return nullptr;
  }
  void* p = scratch_address[dev].load(std::memory_order_acquire);
  if (p) return p;
  e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) {
    *err = e != hipSuccess ? e : hipErrorInvalidSymbol;
    return nullptr;
  }
  scratch_address[dev].store(p, std::memory_order_release);  // (racing threads store the same value)
  return p;
}

// ---- workspace the plain entry points hold themselves -------------------------------------------
// adr_matmul_f16, adr_matmul_nt_f16 and adr_matmul_nt_fp16u8 have the reference's argument tuples
// and therefore no workspace argument.  Where a workspace pays (K split over workgroups; on request
// the u8 matrix dequantised once) they take it from a pool that grows on demand.  A buffer has an
// owner, (device, stream) -- launches on one stream run in order, launches on different streams may
// overlap -- and an event recorded behind the last launches that used it.  A buffer changes hands
// (a buffer its owner outgrew, or the least recently used one when all MAX_HELD entries are
// taken) by making the new owner's stream wait for that event: no host synchronisation, no free
// and no allocation inside a matmul call beyond the first ones.  Memory goes back to the device
// only through adr_release_held_workspace*, which wait for the event first.
constexpr int MAX_HELD = 16;
constexpr int64_t HELD_FLOOR = (int64_t)16 << 20;
struct Held {
  int device;
  hipStream_t stream;  // owner; `owned` false: outgrown by its owner, free to be taken over
  bool owned;
  void* ptr;
  int64_t bytes;
  hipEvent_t last_use;  // recorded on the owner's stream behind the last launches that used ptr
  uint64_t tick;        // value of held_clock at the last use
};
std::mutex held_mutex;
Held held[MAX_HELD];
int held_count = 0;
int64_t held_total = 0;     // bytes allocated and not yet released
uint64_t held_clock = 0;
std::atomic<int64_t> held_declined{0};  // calls that wanted a buffer and ran without
std::atomic<int64_t> held_limit{ADR_HELD_WORKSPACE_DEFAULT_BYTES};
std::atomic<int> u8_dequantise_first_enabled{0};

// May this call use (and if need be allocate) a held buffer on `stream`?  Not while the stream is
// being captured: the launches would tie the buffer into a graph that can be replayed on any stream
// at any time.  Not on the per-thread default stream, whose handle names a different stream in
// every thread.
bool held_allowed(hipStream_t stream) {
  if (stream == hipStreamPerThread) return false;
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st == hipStreamCaptureStatusNone;
}

// `stream` takes over entry h: everything the previous owner launched on the buffer is ordered
// before whatever `stream` launches next.
bool held_take_over(Held* h, hipStream_t stream) {
  if (hipStreamWaitEvent(stream, h->last_use, 0) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  h->stream = stream;
  h->owned = true;
  return true;
}

// A buffer of at least `want` bytes for (current device, stream), or null (then the caller runs
// without one, and the call is counted in held_declined).  held_mutex is held by the caller, and
// stays held over the launches that use the buffer and the held_used() behind them, so that two
// threads launching on one stream cannot interleave their pairs of launches.
Held* held_buffer(hipStream_t stream, int64_t want) {
  const int64_t limit = held_limit.load(std::memory_order_relaxed);
  if (want <= 0) return nullptr;
  auto declined = [&]() -> Held* {
    held_declined.fetch_add(1, std::memory_order_relaxed);
    return nullptr;
  };
  if (want > limit) return declined();
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return declined();
  Held* mine = nullptr;
  for (int i = 0; i < held_count; i++)
    if (held[i].owned && held[i].device == dev && held[i].stream == stream) mine = &held[i];
  if (mine && mine->bytes >= want) return mine;
  // a buffer some stream outgrew that is large enough
  for (int i = 0; i < held_count; i++)
    if (!held[i].owned && held[i].device == dev && held[i].bytes >= want && held_take_over(&held[i], stream)) {
      if (mine) mine->owned = false;
      return &held[i];
    }
  if (held_count < MAX_HELD) {
    int64_t size = HELD_FLOOR;
    while (size < want) size *= 2;
    if (size > limit) size = limit;
    // (an allocation is an "unsafe" call for a capture in global mode that some other stream of the
    // process may be in; it touches no stream, so it is made in relaxed mode)
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    (void)hipThreadExchangeStreamCaptureMode(&mode);
    void* p = nullptr;
    hipEvent_t ev = nullptr;
    hipError_t e = hipMalloc(&p, (size_t)size);
    if (e == hipSuccess && p) {
      e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
      if (e != hipSuccess) (void)hipFree(p);
    }
    (void)hipThreadExchangeStreamCaptureMode(&mode);
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();  // out of memory: the product runs without a workspace
      return declined();
    }
    if (mine) mine->owned = false;  // outgrown: stays in the pool for a stream that wants less
    Held* h = &held[held_count++];
    *h = Held{dev, stream, true, p, size, ev, 0};
    held_total += size;
    return h;
  }
  // every entry is taken: the least recently used buffer of this device that is large enough
  Held* lru = nullptr;
  for (int i = 0; i < held_count; i++)
    if (held[i].device == dev && held[i].bytes >= want && &held[i] != mine &&
        (!lru || held[i].tick < lru->tick))
      lru = &held[i];
  if (lru && held_take_over(lru, stream)) {
    if (mine) mine->owned = false;
    return lru;
  }
  return declined();
}

// behind the launches that used h->ptr on its owner's stream
void held_used(Held* h) {
  h->tick = ++held_clock;
  if (hipEventRecord(h->last_use, h->stream) != hipSuccess) (void)hipGetLastError();
}

// Frees entry i (waits for its last use first) and closes the gap.  held_mutex is held.
void held_free(int i) {
  (void)hipEventSynchronize(held[i].last_use);
  (void)hipEventDestroy(held[i].last_use);
  (void)hipFree(held[i].ptr);
  (void)hipGetLastError();
  held_total -= held[i].bytes;
  held[i] = held[--held_count];
}

// run_matmul for the entry points without a workspace argument.
int run_matmul_held(hipStream_t stream, MatmulArgs& a) {
  if (empty(a)) return ADR_OK;
  if (int rc = check_device()) return rc;
  const char* name;
  const int64_t limit = held_limit.load(std::memory_order_relaxed);
  // (a product that would like more than the limit is cut into fewer pieces, or not at all)
  const int64_t need = limit > 0 && !gemv_f16_supported(a, &name) ? mfma_gemm_workspace_bytes(a, limit) : 0;
  if (need > 0 && held_allowed(stream)) {
    std::lock_guard<std::mutex> lock(held_mutex);
    if (Held* h = held_buffer(stream, need)) {
      a.workspace = (float*)h->ptr;
      a.workspace_bytes = h->bytes;
      const int rc = run_matmul(stream, a, true);
      held_used(h);
      return rc;
    }
  }
  return run_matmul(stream, a, true);
}

}  // namespace

extern "C" {

int adr_abi_version(void) { return ABI_VERSION; }

const char* adr_strerror(int code) {
  switch (code) {
    case ADR_OK: return "success";
    case ADR_EINVAL_SHAPE: return "invalid shape or size";
    case ADR_EINVAL_ENUM: return "store/load/mask operator out of range";
    case ADR_ENOTIMPL: return "MatmulStoreOp::GeluBias has no device implementation";
    case ADR_ENULL: return "null tensor pointer or missing bias";
    case ADR_EDIVISIBILITY: return "size not divisible by block_size / unsupported block_size";
    case ADR_EUNSUPPORTED_DEVICE: return "current device is not gfx950";
    case ADR_ESCRATCH:
      return "adr_matmul_f16_noalloc: the product would split K with more scratch than the built-in "
             "ADR_NOALLOC_SCRATCH_BYTES; use adr_matmul_f16 or adr_matmul_f16_ws";
    case ADR_EUNSUPPORTED_LAYOUT:
      return "fused attention covers head dimension 64 or 128, unit x strides, y/z strides that "
             "are multiples of 8 and 16-byte aligned pointers";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
  }
}

int adr_matmul_f16(adr_stream_t stream, uint16_t* output, const uint16_t* lhs, const uint16_t* rhs,
                   int32_t batches, int32_t m, int32_t k, int32_t n, int32_t stride_ox,
                   int32_t stride_oy, int32_t stride_oz, int32_t stride_lx, int32_t stride_ly,
                   int32_t stride_lz, int32_t stride_rx, int32_t stride_ry, int32_t stride_rz,
                   const uint16_t* bias, float beta, float scale, uint32_t store, uint32_t load,
                   uint32_t mask) {
  MatmulArgs a = pack(output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                      stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, bias, beta,
                      scale, store, load, mask);
  if (int rc = validate_matmul(a, true)) return rc;
  return run_matmul_held((hipStream_t)stream, a);
}

int adr_set_held_workspace_limit(int64_t bytes) {
  if (bytes < 0) return ADR_EINVAL_SHAPE;
  held_limit.store(bytes, std::memory_order_relaxed);
  return ADR_OK;
}

int64_t adr_held_workspace_limit(void) { return held_limit.load(std::memory_order_relaxed); }

int64_t adr_held_workspace_bytes(void) {
  std::lock_guard<std::mutex> lock(held_mutex);
  return held_total;
}

int64_t adr_held_workspace_declined(void) { return held_declined.load(std::memory_order_relaxed); }

int adr_release_held_workspace(adr_stream_t stream) {
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev)) return (int)e;
  std::lock_guard<std::mutex> lock(held_mutex);
  for (int i = held_count - 1; i >= 0; i--)
    if (held[i].device == dev && (!held[i].owned || held[i].stream == (hipStream_t)stream)) held_free(i);
  return ADR_OK;
}

int adr_release_held_workspace_all(void) {
  std::lock_guard<std::mutex> lock(held_mutex);
  while (held_count > 0) held_free(held_count - 1);
  return ADR_OK;
}

int adr_set_u8_dequantise_first(int enabled) {
  u8_dequantise_first_enabled.store(enabled != 0, std::memory_order_relaxed);
  return ADR_OK;
}

int adr_u8_dequantise_first(void) { return u8_dequantise_first_enabled.load(std::memory_order_relaxed); }

int adr_matmul_f16_ws(adr_stream_t stream, uint16_t* output, const uint16_t* lhs, const uint16_t* rhs,
                      int32_t batches, int32_t m, int32_t k, int32_t n, int32_t stride_ox,
                      int32_t stride_oy, int32_t stride_oz, int32_t stride_lx, int32_t stride_ly,
                      int32_t stride_lz, int32_t stride_rx, int32_t stride_ry, int32_t stride_rz,
                      const uint16_t* bias, float beta, float scale, uint32_t store, uint32_t load,
                      uint32_t mask, void* workspace, int64_t workspace_bytes) {
  MatmulArgs a = pack(output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                      stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, bias, beta,
                      scale, store, load, mask);
  if (int rc = validate_matmul(a, true)) return rc;
  if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return ADR_ENULL;
  if ((uintptr_t)workspace % 16 != 0) return ADR_EINVAL_SHAPE;
  a.workspace = (float*)workspace;
  a.workspace_bytes = workspace_bytes;
  return run_matmul((hipStream_t)stream, a, true);
}

int adr_matmul_f16_noalloc(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                           const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                           int32_t stride_ox, int32_t stride_oy, int32_t stride_oz, int32_t stride_lx,
                           int32_t stride_ly, int32_t stride_lz, int32_t stride_rx, int32_t stride_ry,
                           int32_t stride_rz, const uint16_t* bias, float beta, float scale,
                           uint32_t store, uint32_t load, uint32_t mask) {
  MatmulArgs a = pack(output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                      stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, bias, beta,
                      scale, store, load, mask);
  if (int rc = validate_matmul(a, true)) return rc;
  if (empty(a)) return ADR_OK;
  if (int rc = check_device()) return rc;
  // what the product uses of the built-in scratch: a product that would like more is cut into
  // fewer pieces, or not at all (the launcher makes the same choice from a.workspace_bytes)
  const char* name;
  const int64_t need =
      gemv_f16_supported(a, &name) ? 0 : mfma_gemm_workspace_bytes(a, ADR_NOALLOC_SCRATCH_BYTES);
  if (need > ADR_NOALLOC_SCRATCH_BYTES) return ADR_ESCRATCH;  // (cannot happen: the choice is bounded)
  if (need > 0) {
    hipError_t e;
    void* p = scratch_on_current_device(&e);
    if (!p) return (int)e;
    a.workspace = (float*)p;
    a.workspace_bytes = ADR_NOALLOC_SCRATCH_BYTES;
  }
  return run_matmul((hipStream_t)stream, a, true);
}

int64_t adr_matmul_f16_workspace_bytes(int32_t batches, int32_t m, int32_t k, int32_t n,
                                       int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                                       int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                                       int32_t stride_rx, int32_t stride_ry, int32_t stride_rz,
                                       uint32_t store, uint32_t load, uint32_t mask) {
  MatmulArgs a = pack(nullptr, nullptr, nullptr, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                      stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, nullptr,
                      0.0f, 1.0f, store, load, mask);
  if (int rc = validate_matmul(a, false)) return rc;
  const char* name;
  if (empty(a) || gemv_f16_supported(a, &name)) return 0;
  return mfma_gemm_workspace_bytes(a);
}

int adr_matmul_f16_slow(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                        const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                        int32_t stride_ox, int32_t stride_oy, int32_t stride_oz, int32_t stride_lx,
                        int32_t stride_ly, int32_t stride_lz, int32_t stride_rx, int32_t stride_ry,
                        int32_t stride_rz, const uint16_t* bias, float beta, float scale,
                        uint32_t store, uint32_t load, uint32_t mask) {
  MatmulArgs a = pack(output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                      stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, bias, beta,
                      scale, store, load, mask);
  if (int rc = validate_matmul(a, true)) return rc;
  return run_matmul((hipStream_t)stream, a, false);
}

int adr_matmul_f16_raw(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                       const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                       int32_t stride_ox, int32_t stride_oy, int32_t stride_oz, int32_t stride_lx,
                       int32_t stride_ly, int32_t stride_lz, int32_t stride_rx, int32_t stride_ry,
                       int32_t stride_rz) {
  return adr_matmul_f16(stream, output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy,
                        stride_oz, stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz,
                        nullptr, 0.0f, 1.0f, ADR_STORE_IDENTITY, ADR_LOAD_IDENTITY, ADR_MASK_NONE);
}

int adr_matmul_f16_plan(char* name, int32_t cap, int32_t batches, int32_t m, int32_t k, int32_t n,
                        int32_t stride_ox, int32_t stride_oy, int32_t stride_oz, int32_t stride_lx,
                        int32_t stride_ly, int32_t stride_lz, int32_t stride_rx, int32_t stride_ry,
                        int32_t stride_rz, uint32_t store, uint32_t load, uint32_t mask) {
  MatmulArgs a = pack(nullptr, nullptr, nullptr, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                      stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, nullptr,
                      0.0f, 1.0f, store, load, mask);
  if (int rc = validate_matmul(a, false)) return rc;
  // what run_matmul_held does on a stream that is not being captured: a workspace of up to the
  // current limit from the library's own pool
  a.workspace_bytes = held_limit.load(std::memory_order_relaxed);
  const char* chosen = "none (empty)";
  if (!empty(a) && !gemv_f16_supported(a, &chosen) && !mfma_gemm_supported(a, &chosen))
    chosen = "matmul_general";
  if (name && cap > 0) {
    strncpy(name, chosen, (size_t)cap - 1);
    name[cap - 1] = 0;
  }
  return ADR_OK;
}

int adr_matmul_f16_ws_plan(char* name, int32_t cap, int32_t batches, int32_t m, int32_t k, int32_t n,
                           int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                           int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                           int32_t stride_rx, int32_t stride_ry, int32_t stride_rz, uint32_t store,
                           uint32_t load, uint32_t mask, int64_t workspace_bytes) {
  MatmulArgs a = pack(nullptr, nullptr, nullptr, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                      stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, nullptr,
                      0.0f, 1.0f, store, load, mask);
  if (int rc = validate_matmul(a, false)) return rc;
  if (workspace_bytes < 0) return ADR_EINVAL_SHAPE;
  a.workspace_bytes = workspace_bytes;
  const char* chosen = "none (empty)";
  if (!empty(a) && !gemv_f16_supported(a, &chosen) && !mfma_gemm_supported(a, &chosen))
    chosen = "matmul_general";
  if (name && cap > 0) {
    strncpy(name, chosen, (size_t)cap - 1);
    name[cap - 1] = 0;
  }
  return ADR_OK;
}

// adr_matmul_nt_f16; `held`: may take the split-K workspace from the library's own cache
static int nt_f16(adr_stream_t stream, uint16_t* output, const uint16_t* lhs, const uint16_t* rhs,
                  int32_t m, int32_t p, int32_t n, float beta, bool held) {
  if (m < 0 || p < 0 || n < 0) return ADR_EINVAL_SHAPE;
  if (m == 0 || n == 0) return ADR_OK;
  if (!output || (p && (!lhs || !rhs))) return ADR_ENULL;
  if ((int64_t)m * n >= ((int64_t)1 << 31) || (int64_t)m * p >= ((int64_t)1 << 31) ||
      (int64_t)n * p >= ((int64_t)1 << 31))
    return ADR_EINVAL_SHAPE;  // (32-bit element offsets, as in adr_matmul_f16)
  MatmulArgs a = pack(output, lhs, rhs, 1, m, p, n, 1, n, 0, 1, p, 0, p, 1, 0, nullptr, beta, 1.0f,
                      STORE_ACC_BETA, ADR_LOAD_IDENTITY, ADR_MASK_NONE);
  return held ? run_matmul_held((hipStream_t)stream, a) : run_matmul((hipStream_t)stream, a, true);
}

int adr_matmul_nt_f16(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                      const uint16_t* rhs, int32_t m, int32_t p, int32_t n, float beta) {
  return nt_f16(stream, output, lhs, rhs, m, p, n, beta, true);
}

// Where dequantising the matrix once and running the fp16 kernels beats the fused kernels
// (measured over M 64 .. 4096 on (K, N) of the LLaMA-7B and 13B layers): from 768 rows on.  Below,
// the fused kernel's small tiles are 5-80 % ahead (K11008 N4096 M512 73 against 84 us, M256 46
// against 63; K4096 N12288 M128 31 against 50); at 768 and 1024 rows the two are within 5 % of each
// other either way; from 1536 rows on the fused kernel dequantises every weight six times and more
// and is 6-25 % behind (K4096 N12288 M2048 218 against 185 us).
static bool u8_dequantise_first(int m, int p, int n) {
  (void)n;
  return m >= 768 && p > 0;
}

static int validate_u8(const uint16_t* output, const uint16_t* lhs, const uint8_t* rhs,
                       const uint16_t* scales, int32_t m, int32_t p, int32_t n, int32_t block_size,
                       bool* nothing_to_do) {
  *nothing_to_do = false;
  if (m < 0 || p < 0 || n < 0 || block_size <= 0) return ADR_EINVAL_SHAPE;
  if (p % block_size != 0) return ADR_EDIVISIBILITY;
  if (m == 0 || n == 0) {
    *nothing_to_do = true;
    return ADR_OK;
  }
  if (!output || (p && (!lhs || !rhs || !scales))) return ADR_ENULL;
  if ((int64_t)m * n >= ((int64_t)1 << 31) || (int64_t)m * p >= ((int64_t)1 << 31) ||
      (int64_t)n * p >= ((int64_t)1 << 31))
    return ADR_EINVAL_SHAPE;  // (32-bit element offsets, as in adr_matmul_f16)
  return ADR_OK;
}

// the matrix dequantised into `workspace` (n * p halves), then the fp16 kernels on it
static int u8_by_way_of_fp16(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                             const uint8_t* rhs, const uint16_t* scales, int32_t m, int32_t p,
                             int32_t n, int32_t block_size, float beta, void* workspace) {
  if (int rc = adr_dequantize_absmax_u8(stream, (uint16_t*)workspace, rhs, scales, n, p, block_size)) return rc;
  return nt_f16(stream, output, lhs, (const uint16_t*)workspace, m, p, n, beta, false);
}

static int u8_fused(adr_stream_t stream, uint16_t* output, const uint16_t* lhs, const uint8_t* rhs,
                    const uint16_t* scales, int32_t m, int32_t p, int32_t n, int32_t block_size,
                    float beta) {
  if (int rc = check_device()) return rc;
  return (int)launch_gemm_u8((hipStream_t)stream, (half_t*)output, (const half_t*)lhs, rhs,
                             (const half_t*)scales, m, p, n, block_size, beta);
}

// Does the plain u8 entry point dequantise first?  Only on request (adr_set_u8_dequantise_first),
// where that is the faster route and the matrix fits the held-workspace limit.
static bool u8_held_route(int m, int p, int n) {
  return u8_dequantise_first_enabled.load(std::memory_order_relaxed) && u8_dequantise_first(m, p, n) &&
         (int64_t)n * p * 2 <= held_limit.load(std::memory_order_relaxed);
}

int adr_matmul_nt_fp16u8(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                         const uint8_t* rhs, const uint16_t* scales, int32_t m, int32_t p,
                         int32_t n, int32_t block_size, float beta) {
  bool nothing;
  if (int rc = validate_u8(output, lhs, rhs, scales, m, p, n, block_size, &nothing)) return rc;
  if (nothing) return ADR_OK;
  if (u8_held_route(m, p, n) && held_allowed((hipStream_t)stream)) {
    if (int rc = check_device()) return rc;
    std::lock_guard<std::mutex> lock(held_mutex);
    if (Held* h = held_buffer((hipStream_t)stream, (int64_t)n * p * 2)) {
      const int rc = u8_by_way_of_fp16(stream, output, lhs, rhs, scales, m, p, n, block_size, beta, h->ptr);
      held_used(h);
      return rc;
    }
  }
  return u8_fused(stream, output, lhs, rhs, scales, m, p, n, block_size, beta);
}

int64_t adr_matmul_nt_fp16u8_workspace_bytes(int32_t m, int32_t p, int32_t n, int32_t block_size) {
  if (m < 0 || p < 0 || n < 0 || block_size <= 0) return ADR_EINVAL_SHAPE;
  if (p % block_size != 0) return ADR_EDIVISIBILITY;
  return u8_dequantise_first(m, p, n) ? (int64_t)n * p * 2 : 0;
}

int adr_matmul_nt_fp16u8_ws(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                            const uint8_t* rhs, const uint16_t* scales, int32_t m, int32_t p,
                            int32_t n, int32_t block_size, float beta, void* workspace,
                            int64_t workspace_bytes) {
  if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return ADR_ENULL;
  if ((uintptr_t)workspace % 16 != 0) return ADR_EINVAL_SHAPE;
  bool nothing;
  if (int rc = validate_u8(output, lhs, rhs, scales, m, p, n, block_size, &nothing)) return rc;
  if (nothing) return ADR_OK;
  // (only the caller's buffer is ever used here, never the library's own)
  if (!u8_dequantise_first(m, p, n) || workspace_bytes < (int64_t)n * p * 2)
    return u8_fused(stream, output, lhs, rhs, scales, m, p, n, block_size, beta);
  return u8_by_way_of_fp16(stream, output, lhs, rhs, scales, m, p, n, block_size, beta, workspace);
}

int adr_matmul_nt_fp16u8_plan(char* name, int32_t cap, int32_t m, int32_t p, int32_t n,
                              int32_t block_size) {
  if (m < 0 || p < 0 || n < 0 || block_size <= 0) return ADR_EINVAL_SHAPE;
  if (p % block_size != 0) return ADR_EDIVISIBILITY;
  const char* chosen = (m == 0 || n == 0) ? "none (empty)" : gemm_u8_plan(m, p, n, block_size);
  // (the opt-in route of the plain entry point on a stream that is not being captured)
  if (m != 0 && n != 0 && u8_held_route(m, p, n)) chosen = "dequantize_absmax_u8 + fp16 gemm";
  if (name && cap > 0) {
    strncpy(name, chosen, (size_t)cap - 1);
    name[cap - 1] = 0;
  }
  return ADR_OK;
}

int adr_dequantize_absmax_uint8(adr_stream_t stream, adr_tensor_desc output,
                                adr_tensor_desc scales, adr_tensor_desc input) {
  if (int rc = validate_quant(output, scales, input)) return rc;
  if (output.shape[0] == 0 || output.shape[1] == 0) return ADR_OK;
  if (int rc = check_device()) return rc;
  return (int)launch_dequantize((hipStream_t)stream, output, scales, input);
}

int adr_quantize_absmax_uint8(adr_stream_t stream, adr_tensor_desc output, adr_tensor_desc scales,
                              adr_tensor_desc input) {
  if (int rc = validate_quant(output, scales, input)) return rc;
  if (output.shape[0] == 0 || output.shape[1] == 0) return ADR_OK;
  if (int rc = check_device()) return rc;
  return (int)launch_quantize((hipStream_t)stream, output, scales, input);
}

int adr_dequantize_absmax_u8(adr_stream_t stream, uint16_t* output, const uint8_t* q,
                             const uint16_t* scales, int32_t rows, int32_t cols,
                             int32_t block_size) {
  if (rows < 0 || cols < 0 || block_size <= 0) return ADR_EINVAL_SHAPE;
  if (cols % block_size != 0) return ADR_EDIVISIBILITY;
  if (rows == 0 || cols == 0) return ADR_OK;
  return adr_dequantize_absmax_uint8(stream, desc2d(output, rows, cols),
                                     desc2d(scales, rows, cols / block_size),
                                     desc2d(q, rows, cols));
}

int adr_quantize_absmax_u8(adr_stream_t stream, uint8_t* q, uint16_t* scales,
                           const uint16_t* input, int32_t rows, int32_t cols, int32_t block_size) {
  if (rows < 0 || cols < 0 || block_size <= 0) return ADR_EINVAL_SHAPE;
  if (cols % block_size != 0) return ADR_EDIVISIBILITY;
  if (rows == 0 || cols == 0) return ADR_OK;
  return adr_quantize_absmax_uint8(stream, desc2d(q, rows, cols),
                                   desc2d(scales, rows, cols / block_size),
                                   desc2d(input, rows, cols));
}

int adr_embed_uint8(adr_stream_t stream, int32_t n_dim, int32_t n_ids, const int16_t* in_ids,
                    uint16_t* out_embeddings, const uint8_t* embeddings_table,
                    const uint16_t* scales, int32_t block_size) {
  if (n_dim < 0 || n_ids < 0 || block_size <= 0) return ADR_EINVAL_SHAPE;
  if (n_dim % block_size != 0) return ADR_EDIVISIBILITY;
  if (n_dim == 0 || n_ids == 0) return ADR_OK;
  if (!in_ids || !out_embeddings || !embeddings_table || !scales) return ADR_ENULL;
  if (int rc = check_device()) return rc;
  return (int)launch_embed_u8((hipStream_t)stream, n_dim, n_ids, in_ids, (half_t*)out_embeddings,
                              embeddings_table, (const half_t*)scales, block_size);
}

int adr_softmax_rows(adr_stream_t stream, uint16_t* output, const uint16_t* input, int32_t heads,
                     int32_t h, int32_t w, float temp) {
  if (heads < 0 || h < 0 || w < 0) return ADR_EINVAL_SHAPE;
  if (heads == 0 || h == 0 || w == 0) return ADR_OK;
  if (!output || !input) return ADR_ENULL;
  if (int rc = check_device()) return rc;
  return (int)launch_softmax_rows((hipStream_t)stream, (half_t*)output, (const half_t*)input,
                                  (int64_t)heads * h, w, temp);
}

int adr_attention_f16(adr_stream_t stream, uint16_t* output, const uint16_t* query,
                      const uint16_t* key, const uint16_t* value, int32_t heads, int32_t m,
                      int32_t n, int32_t d, int32_t stride_ox, int32_t stride_oy,
                      int32_t stride_oz, int32_t stride_qx, int32_t stride_qy, int32_t stride_qz,
                      int32_t stride_kx, int32_t stride_ky, int32_t stride_kz, int32_t stride_vx,
                      int32_t stride_vy, int32_t stride_vz, float scale, float temp,
                      uint32_t mask) {
  if (heads < 0 || m < 0 || n < 0 || d < 0) return ADR_EINVAL_SHAPE;
  if (mask > ADR_MASK_CAUSAL) return ADR_EINVAL_ENUM;
  if (heads == 0 || m == 0 || d == 0) return ADR_OK;
  if (n == 0) return ADR_EINVAL_SHAPE;
  if (!output || !query || !key || !value) return ADR_ENULL;
  if (d != 64 && d != 128) return ADR_EUNSUPPORTED_LAYOUT;
  if (stride_ox != 1 || stride_qx != 1 || stride_kx != 1 || stride_vx != 1)
    return ADR_EUNSUPPORTED_LAYOUT;
  const int32_t st[8] = {stride_oy, stride_oz, stride_qy, stride_qz,
                         stride_ky, stride_kz, stride_vy, stride_vz};
  for (int i = 0; i < 8; i++)
    if (st[i] < 0 || st[i] % 8 != 0) return ADR_EUNSUPPORTED_LAYOUT;
  if (((uintptr_t)output | (uintptr_t)query | (uintptr_t)key | (uintptr_t)value) % 16 != 0)
    return ADR_EUNSUPPORTED_LAYOUT;
  if (!(scale > 0.0f) || !(temp > 0.0f)) return ADR_EUNSUPPORTED_LAYOUT;
  // largest element offsets stay within int64 trivially; rows are addressed with 64-bit products
  if (int rc = check_device()) return rc;
  return (int)launch_attention((hipStream_t)stream, (half_t*)output, (const half_t*)query,
                               (const half_t*)key, (const half_t*)value, heads, m, n, d,
                               stride_oy, stride_oz, stride_qy, stride_qz, stride_ky, stride_kz,
                               stride_vy, stride_vz, scale, temp, mask);
}

static int error_stats_common(adr_stream_t stream, adr_tensor_desc output, adr_tensor_desc lhs,
                              adr_tensor_desc rhs, bool f32) {
  if (output.dims != 1 || lhs.dims != 1 || rhs.dims != 1) return ADR_EINVAL_SHAPE;
  if (output.shape[0] < 3 || output.strides[0] != 1 || lhs.shape[0] != rhs.shape[0])
    return ADR_EINVAL_SHAPE;
  if (lhs.shape[0] == 0) return ADR_OK;
  if (!output.ptr || !lhs.ptr || !rhs.ptr) return ADR_ENULL;
  if (int rc = check_device()) return rc;
  return (int)launch_error_stats((hipStream_t)stream, (float*)output.ptr, lhs.ptr, rhs.ptr,
                                 lhs.shape[0], lhs.strides[0], rhs.strides[0], f32);
}

int adr_debug_knob(int32_t id, int32_t value) { return set_knob(id, value); }

int adr_microbench_empty(adr_stream_t stream) {
  if (int rc = check_device()) return rc;
  return (int)launch_microbench_empty((hipStream_t)stream);
}

int adr_microbench_mfma_f16(adr_stream_t stream, int blocks, int times, int pattern, float* sink) {
  if (blocks <= 0 || times < 0 || pattern < 0 || pattern > 4) return ADR_EINVAL_SHAPE;
  if (!sink) return ADR_ENULL;
  if (int rc = check_device()) return rc;
  return (int)launch_microbench_mfma((hipStream_t)stream, blocks, times, pattern, sink);
}

int adr_microbench_stream_read(adr_stream_t stream, const void* src, int64_t bytes, int blocks,
                               uint32_t* sink) {
  if (blocks <= 0 || bytes < 0 || bytes % (16 * (int64_t)blocks) != 0) return ADR_EINVAL_SHAPE;
  if (bytes == 0) return ADR_OK;
  if (!src || !sink) return ADR_ENULL;
  if ((uintptr_t)src % 16 != 0) return ADR_EINVAL_SHAPE;
  if (int rc = check_device()) return rc;
  return (int)launch_microbench_read((hipStream_t)stream, src, bytes, blocks, sink);
}

int adr_error_stats_f16(adr_stream_t stream, adr_tensor_desc output, adr_tensor_desc lhs,
                        adr_tensor_desc rhs) {
  return error_stats_common(stream, output, lhs, rhs, false);
}

int adr_error_stats_f32(adr_stream_t stream, adr_tensor_desc output, adr_tensor_desc lhs,
                        adr_tensor_desc rhs) {
  return error_stats_common(stream, output, lhs, rhs, true);
}

}  // extern "C"
