// The runtime behind the C ABI (include/vkt.h): one device, one caching memory pool, one
// in-order HIP stream, and a table of named kernels.  It takes the place of the
// reference's Rust core (crates/vkcore/src/lib.rs:33-76 `Runtime`, context.rs, memory.rs,
// kernels.rs, stream.rs) and its C ABI (crates/pyvk/src/ffi.rs).
//
// HIP gives for free what the reference builds by hand on Vulkan: a stream is in order
// (no barriers to place, stream.rs:116-176), code objects are compiled ahead of time
// (no pipeline cache, kernels.rs:72-154), and device pointers are plain addresses (no
// address map, backend.cpp:170-192).  What stays is policy: the pool, the error
// convention, lazy start-up and safe shutdown.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>

#include "../../../include/vkt.h"
#include "../kernels/kernels.h"
#include "pool.h"

namespace vkt {
namespace {

thread_local std::string g_last_error;

int fail(const std::string& message) {
  g_last_error = message;
  for (char& c : g_last_error)
    if (c == '\0') c = ' ';
  return -1;
}

std::string hip_message(const char* what, hipError_t e) {
  return std::string(what) + ": " + hipGetErrorString(e) + " (" + hipGetErrorName(e) + ")";
}

struct HipSource {
  bool map(uint64_t bytes, uint64_t* address, std::string* err) {
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
      (void)hipGetLastError();  // clear the sticky out-of-memory status
      *err = hip_message("hipMalloc", e) + " for " + std::to_string(bytes) + " bytes";
      return false;
    }
    *address = reinterpret_cast<uint64_t>(p);
    return true;
  }
  void unmap(uint64_t address) { (void)hipFree(reinterpret_cast<void*>(address)); }
};

struct Runtime {
  int device = 0;
  hipDeviceProp_t props{};
  Machine machine;
  hipStream_t stream = nullptr;
  std::mutex pool_mutex;  // lock order: pool, then stream (vkcore/src/lib.rs:33-50)
  std::mutex stream_mutex;
  std::unique_ptr<Pool<HipSource>> pool;
  std::atomic<uint64_t> dispatches{0};
  bool trace = false;
  uint64_t generation = 0;
  void* workspace_base = nullptr;
  void* scratch_base = nullptr;

  // Grows the scratch region to at least `bytes` (never shrinks before vkt_empty_cache / shutdown).  hipFree waits
  // for the device, so a region still in use by queued kernels is not pulled away.  Caller holds stream_mutex.
  bool ensure_scratch(uint64_t bytes, std::string* err) {
    if (bytes <= machine.scratch_bytes) return true;
    if (scratch_base) (void)hipFree(scratch_base);
    scratch_base = nullptr, machine.scratch = 0, machine.scratch_bytes = 0;
    const uint64_t want = (bytes + (uint64_t(64) << 20) - 1) >> 26 << 26;  // whole 64 MiB
    void* base = nullptr;
    const hipError_t e = hipMalloc(&base, want);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      *err = hip_message("scratch allocation", e);
      return false;
    }
    scratch_base = base, machine.scratch = reinterpret_cast<uint64_t>(base), machine.scratch_bytes = want;
    return true;
  }
  void drop_scratch() {
    if (scratch_base) (void)hipFree(scratch_base);
    scratch_base = nullptr, machine.scratch = 0, machine.scratch_bytes = 0;
  }

  ~Runtime() {
    if (stream) {
      (void)hipStreamSynchronize(stream);
    }
    pool.reset();
    if (workspace_base) (void)hipFree(workspace_base);
    if (scratch_base) (void)hipFree(scratch_base);
    if (stream) (void)hipStreamDestroy(stream);
  }
};

std::mutex g_mutex;
std::shared_ptr<Runtime> g_runtime;
uint64_t g_generation = 0;

void idle_hook(void* arg) {
  Runtime* rt = static_cast<Runtime*>(arg);
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  (void)hipStreamSynchronize(rt->stream);
}

// Starts the runtime on first use (reference pyvk/src/lib.rs:18-24).
std::shared_ptr<Runtime> runtime(std::string* err) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_runtime) return g_runtime;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0) {
    (void)hipGetLastError();
    *err = e != hipSuccess ? hip_message("no usable GPU: hipGetDeviceCount", e) : "no usable GPU: no HIP device";
    return nullptr;
  }
  auto rt = std::make_shared<Runtime>();
  const char* dev = std::getenv("VKT_DEVICE");
  rt->device = dev ? std::atoi(dev) : 0;
  if (rt->device < 0 || rt->device >= count) {
    *err = "VKT_DEVICE out of range";
    return nullptr;
  }
  if ((e = hipSetDevice(rt->device)) != hipSuccess || (e = hipGetDeviceProperties(&rt->props, rt->device)) != hipSuccess) {
    *err = hip_message("device start-up", e);
    return nullptr;
  }
  if (std::strncmp(rt->props.gcnArchName, "gfx950", 6) != 0) {
    *err = std::string("this library holds gfx950 (MI355X) code only; device 0 is ") + rt->props.gcnArchName;
    return nullptr;
  }
  // A blocking stream: ordered against the legacy default stream, so a host program that
  // also uses the default stream (PyTorch-ROCm does) needs no extra events.
  if ((e = hipStreamCreateWithFlags(&rt->stream, hipStreamDefault)) != hipSuccess) {
    *err = hip_message("hipStreamCreate", e);
    return nullptr;
  }
  rt->machine.compute_units = rt->props.multiProcessorCount;
  // The kernels' own workspace (partial tiles of products that are split over workgroups).
  // Held outside the pool until shutdown: it is not the caller's memory and does not show
  // in vkt_memory_stats.  Every use is queued on the runtime's one stream, so uses do not
  // overlap.
  {
    constexpr uint64_t kWorkspaceBytes = 32ull << 20;
    void* base = nullptr;
    if ((e = hipMalloc(&base, kWorkspaceBytes)) != hipSuccess) {
      *err = hip_message("workspace allocation", e);
      return nullptr;
    }
    rt->workspace_base = base;
    rt->machine.workspace = reinterpret_cast<uint64_t>(base);
    rt->machine.workspace_bytes = kWorkspaceBytes;
  }
  rt->pool = std::make_unique<Pool<HipSource>>(HipSource{});
  rt->pool->set_idle_hook(&idle_hook, rt.get());
  const char* tr = std::getenv("TORCH_VK_TRACE");  // reference ffi.rs:144-148
  rt->trace = tr && *tr && std::strcmp(tr, "0") != 0;
  rt->generation = ++g_generation;
  g_runtime = rt;
  return rt;
}

std::shared_ptr<Runtime> running() {
  std::lock_guard<std::mutex> lock(g_mutex);
  return g_runtime;
}

int dtype_of_suffix(const char* suffix) {
  if (!std::strcmp(suffix, "f32")) return VKT_F32;
  if (!std::strcmp(suffix, "f16")) return VKT_F16;
  if (!std::strcmp(suffix, "bf16")) return VKT_BF16;
  return -1;
}

template <class P>
bool read_push(const uint8_t* push, size_t npush, P* out, const char* name, std::string* err) {
  if (npush != sizeof(P)) {
    *err = std::string("kernel ") + name + " takes a parameter block of " + std::to_string(sizeof(P)) + " bytes, got " +
           std::to_string(npush);
    return false;
  }
  std::memcpy(out, push, sizeof(P));
  return true;
}

// name + specialisation constants -> launcher (the role of kernels.rs:72-140 KernelCache::get).
int dispatch_named(Runtime& rt, const char* name, const uint32_t* spec, size_t nspec, const uint8_t* push, size_t npush,
                   uint32_t gz, std::string* err) {
  auto spec_at = [&](size_t i) { return i < nspec ? spec[i] : 0u; };
  if (!std::strncmp(name, "qmm8_", 5)) {
    int dt = dtype_of_suffix(name + 5);
    Q8Params p;
    if (dt < 0) goto unknown;
    if (!read_push(push, npush, &p, name, err)) return -1;
    // spec[0] is the reference's ROWS constant (0: tile path, 1..8: GEMV); the row count
    // that matters is p.m, so it is checked for consistency only.
    if (spec_at(0) != 0 && spec_at(0) != p.m) {
      *err = "qmm8: specialisation ROWS=" + std::to_string(spec_at(0)) + " does not match m=" + std::to_string(p.m);
      return -1;
    }
    // (many rows: the weights are widened into the scratch region first; without memory for it the row-block kernels run)
    if (const uint64_t need = q8_gemm_scratch_bytes(p, dt, rt.machine); need != 0 && !((spec_at(1) >> 20) & 1)) {
      std::string ignored;
      (void)rt.ensure_scratch(need, &ignored);
    }
    return launch_qmm8(p, dt, spec_at(1), rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "qmm4_packvec")) {
    Q4VecParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_qmm4_packvec(p, rt.stream, err);
  }
  if (!std::strncmp(name, "qmm4_", 5)) {
    int dt = dtype_of_suffix(name + 5);
    Q4Params p;
    if (dt != VKT_F32 && dt != VKT_BF16) goto unknown;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_qmm4(p, dt, spec_at(0), spec_at(1), rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "qmm4c_pack")) {
    Q4PackParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_qmm4c_pack(p, spec_at(0), rt.machine, rt.stream, err);
  }
  if (!std::strncmp(name, "qmm4c_", 6)) {
    int dt = dtype_of_suffix(name + 6);
    Q4CParams p;
    if (dt != VKT_F32 && dt != VKT_BF16) goto unknown;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_qmm4c(p, dt, spec_at(0), spec_at(1), spec_at(2), rt.machine, rt.stream, err);
  }
  if (!std::strncmp(name, "gemmcm_", 7)) {
    int dt = dtype_of_suffix(name + 7);
    GemmParams p;
    if (dt != VKT_BF16 && dt != VKT_F16) goto unknown;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_gemm16(p, dt, spec_at(0), gz, spec_at(3), rt.machine, rt.stream, err);
  }
  if (!std::strncmp(name, "move_", 5)) {
    StridedParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_move(p, name + 5, spec_at(0), spec_at(2), rt.machine, rt.stream, err);
  }
  if (!std::strncmp(name, "copy8_", 6)) {
    Copy8Params p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_copy8(p, name + 6, spec_at(0), rt.machine, rt.stream, err);
  }
  if (!std::strncmp(name, "cast_", 5) && std::strcmp(name, "cast_fp8")) {
    // "cast_<src>_<dst>"
    const char* second = std::strchr(name + 5, '_');
    if (!second) goto unknown;
    const std::string from(name + 5, second);
    const int sdt = dtype_of_suffix(from.c_str()), ddt = dtype_of_suffix(second + 1);
    StridedParams p;
    if (sdt < 0 || ddt < 0 || sdt == ddt) goto unknown;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_cast_strided(p, sdt, ddt, rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "cast_fp8")) {
    CastParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_cast_fp8(p, rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "quantize_affine") || !std::strcmp(name, "dequantize_affine")) {
    QuantParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_quantize_affine(p, spec_at(0), name[0] == 'd', rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "aminmax")) {
    MinMaxParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_aminmax(p, rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "fake_quant") || !std::strcmp(name, "aminmax")) {
    QuantParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_fake_quant(p, spec_at(0), spec_at(1), rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "fp8_quant") || !std::strncmp(name, "move_", 5) || !std::strncmp(name, "copy8_", 6) ||
          !std::strncmp(name, "cast_", 5) || !std::strcmp(name, "quantize_affine") || !std::strcmp(name, "dequantize_affine") ||
          !std::strcmp(name, "fake_quant") || !std::strcmp(name, "aminmax")) {
    F8QuantParams p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_fp8_quant(p, spec_at(0), rt.machine, rt.stream, err);
  }
  if (!std::strcmp(name, "fp8mm")) {
    F8Params p;
    if (!read_push(push, npush, &p, name, err)) return -1;
    return launch_fp8mm(p, spec_at(0), rt.machine, rt.stream, err);
  }
unknown:
  *err = std::string("unknown kernel ") + name;
  return -1;
}

struct Handle {
  Allocation a;
  uint64_t generation;  // of the runtime that made it: a handle outliving a shutdown is only deleted
};

}  // namespace
}  // namespace vkt

using namespace vkt;

extern "C" {

const char* vkt_last_error(void) { return g_last_error.c_str(); }

int vkt_alloc(uint64_t nbytes, VktAlloc* out) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (!out) return fail("vkt_alloc: null output");
  Allocation a;
  {
    std::lock_guard<std::mutex> lock(rt->pool_mutex);
    if (!rt->pool->alloc(nbytes, &a, &err)) return fail(err);
  }
  out->handle = new Handle{a, rt->generation};
  out->host = nullptr;
  out->address = a.address;
  out->size = a.size;
  return 0;
}

void vkt_free(void* handle) {
  if (!handle) return;
  std::unique_ptr<Handle> h(static_cast<Handle*>(handle));
  auto rt = running();
  if (rt && rt->generation == h->generation) {
    std::lock_guard<std::mutex> lock(rt->pool_mutex);
    rt->pool->free(h->a);
  }
}

int vkt_synchronize(void) {
  auto rt = running();
  if (!rt) return 0;
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  hipError_t e = hipStreamSynchronize(rt->stream);
  return e == hipSuccess ? 0 : fail(hip_message("hipStreamSynchronize", e));
}

int vkt_empty_cache(void) {
  auto rt = running();
  if (!rt) return 0;
  int rc = vkt_synchronize();
  std::lock_guard<std::mutex> lock(rt->pool_mutex);
  rt->pool->trim();
  {
    std::lock_guard<std::mutex> stream_lock(rt->stream_mutex);
    rt->drop_scratch();
  }
  return rc;
}

void vkt_memory_stats(uint64_t* allocated, uint64_t* reserved) {
  uint64_t a = 0, r = 0;
  if (auto rt = running()) {
    std::lock_guard<std::mutex> lock(rt->pool_mutex);
    PoolStats s = rt->pool->stats();
    a = s.allocated;
    r = s.reserved;
  }
  if (allocated) *allocated = a;
  if (reserved) *reserved = r;
}

int vkt_dispatch(const char* name, const uint32_t* spec, size_t nspec, const uint8_t* push, size_t npush, uint32_t gx,
                 uint32_t gy, uint32_t gz) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (!name) return fail("kernel name is null");
  if (npush > 128) return fail("parameter blocks are limited to 128 bytes");
  if (npush != 0 && !push) return fail("parameter block is null");
  if (gx == 0 || gy == 0 || gz == 0) return fail("empty grid");
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  if (dispatch_named(*rt, name, spec, nspec, push, npush, gz, &err) != 0) return fail(err);
  rt->dispatches.fetch_add(1, std::memory_order_relaxed);
  if (rt->trace) {
    // each kernel runs to completion before the next is queued, so a kernel that
    // faults is the last one printed (ffi.rs:135-142)
    std::fprintf(stderr, "[vkt] %s [", name);
    for (size_t i = 0; i < nspec; ++i) std::fprintf(stderr, i ? ", %u" : "%u", spec[i]);
    std::fprintf(stderr, "] grid %ux%ux%u\n", gx, gy, gz);
    std::fflush(stderr);
    hipError_t e = hipStreamSynchronize(rt->stream);
    if (e != hipSuccess) return fail(hip_message(name, e));
  }
  return 0;
}

int vkt_grid_1d(uint64_t n, uint32_t* groups, uint32_t* stride) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  // workgroups of 256 threads; at most 16 per compute unit, the rest by grid stride
  const uint64_t want = (n + 255) / 256, cap = uint64_t(rt->machine.compute_units) * 16;
  const uint64_t g = want < 1 ? 1 : (want < cap ? want : cap);
  if (groups) *groups = static_cast<uint32_t>(g);
  if (stride) *stride = static_cast<uint32_t>(g * 256);
  return 0;
}

int vkt_has_float64(void) {
  std::string err;
  return runtime(&err) ? 1 : 0;
}

uint32_t vkt_vendor_id(void) {
  std::string err;
  return runtime(&err) ? 0x1002u : 0u;
}

uint32_t vkt_capabilities(void) {
  std::string err;
  if (!runtime(&err)) return 0;
  // float64 | int16 | float16 | int8 | >= 32 KiB shared memory (vk.h:92-101); the
  // cooperative-matrix bits describe Vulkan kernels this library does not hold.
  return 1u | 2u | 4u | 8u | 64u;
}

uint32_t vkt_kernel_subgroup_size(const char* name) {
  if (!name) return 0;
  std::string err;
  if (!runtime(&err)) return 0;
  return (!std::strncmp(name, "qmm", 3) || !std::strcmp(name, "fp8mm") || !std::strcmp(name, "cast_fp8") || !std::strncmp(name, "gemmcm_", 7) ||
          !std::strcmp(name, "fp8_quant") || !std::strncmp(name, "move_", 5) || !std::strncmp(name, "copy8_", 6) ||
          !std::strncmp(name, "cast_", 5) || !std::strcmp(name, "quantize_affine") || !std::strcmp(name, "dequantize_affine") ||
          !std::strcmp(name, "fake_quant") || !std::strcmp(name, "aminmax"))
             ? 64u
             : 0u;
}

int vkt_copy_to_device(uint64_t dst, const void* src, uint64_t nbytes) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (nbytes == 0) return 0;
  if (!dst || !src) return fail("vkt_copy_to_device: null address");
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  hipError_t e = hipMemcpyAsync(reinterpret_cast<void*>(dst), src, nbytes, hipMemcpyHostToDevice, rt->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(rt->stream);
  return e == hipSuccess ? 0 : fail(hip_message("copy to device", e));
}

int vkt_copy_to_host(void* dst, uint64_t src, uint64_t nbytes) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (nbytes == 0) return 0;
  if (!dst || !src) return fail("vkt_copy_to_host: null address");
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  hipError_t e = hipMemcpyAsync(dst, reinterpret_cast<const void*>(src), nbytes, hipMemcpyDeviceToHost, rt->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(rt->stream);
  return e == hipSuccess ? 0 : fail(hip_message("copy to host", e));
}

int vkt_copy_on_device(uint64_t dst, uint64_t src, uint64_t nbytes) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (nbytes == 0) return 0;
  if (!dst || !src) return fail("vkt_copy_on_device: null address");
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  // a kernel on the stream (not a DMA engine): it is ordered like every other dispatch, can
  // be recorded into a HIP graph, and shows up in kernel traces and counters
  if (launch_copy(dst, src, nbytes, rt->stream, &err) != 0) return fail(err);
  return 0;
}

int vkt_fill(uint64_t dst, uint8_t value, uint64_t nbytes) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (nbytes == 0) return 0;
  if (!dst) return fail("vkt_fill: null address");
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  // a kernel, not hipMemsetAsync: callers may record this stream into a HIP graph
  if (launch_fill(dst, value, nbytes, rt->stream, &err) != 0) return fail(err);
  return 0;
}

int vkt_device_info(VktDeviceInfo* out) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (!out) return fail("vkt_device_info: null output");
  std::memset(out, 0, sizeof(*out));
  std::strncpy(out->name, rt->props.gcnArchName, sizeof(out->name) - 1);
  out->compute_units = static_cast<uint32_t>(rt->props.multiProcessorCount);
  out->clock_khz = static_cast<uint32_t>(rt->props.clockRate);
  out->mem_clock_khz = static_cast<uint32_t>(rt->props.memoryClockRate);
  out->mem_bus_bits = static_cast<uint32_t>(rt->props.memoryBusWidth);
  out->hbm_bytes = rt->props.totalGlobalMem;
  out->lds_bytes_per_block = static_cast<uint32_t>(rt->props.sharedMemPerBlock);
  out->l2_bytes = static_cast<uint32_t>(rt->props.l2CacheSize);
  return 0;
}

int vkt_event_create(void** event) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (!event) return fail("vkt_event_create: null output");
  hipEvent_t ev;
  hipError_t e = hipEventCreate(&ev);
  if (e != hipSuccess) return fail(hip_message("hipEventCreate", e));
  *event = ev;
  return 0;
}

int vkt_event_record(void* event) {
  auto rt = running();
  if (!rt) return fail("the runtime is not running");
  if (!event) return fail("vkt_event_record: null event");
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  hipError_t e = hipEventRecord(static_cast<hipEvent_t>(event), rt->stream);
  return e == hipSuccess ? 0 : fail(hip_message("hipEventRecord", e));
}

int vkt_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return fail("vkt_event_elapsed_ms: null argument");
  hipError_t e = hipEventSynchronize(static_cast<hipEvent_t>(stop));
  if (e == hipSuccess) e = hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop));
  return e == hipSuccess ? 0 : fail(hip_message("event timing", e));
}

void vkt_event_destroy(void* event) {
  if (event && running()) (void)hipEventDestroy(static_cast<hipEvent_t>(event));
}

uint64_t vkt_dispatch_count(void) {
  auto rt = running();
  return rt ? rt->dispatches.load(std::memory_order_relaxed) : 0;
}

void vkt_shutdown(void) {
  std::shared_ptr<Runtime> rt;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    rt.swap(g_runtime);
  }
  rt.reset();  // waits for queued work, frees the pool's blocks
}

uint64_t vkt_qmm4c_bytes(uint32_t n, uint32_t k, uint32_t bs) { return qmm4c_bytes(n, k, bs); }
uint64_t vkt_qmm4c_q_bytes(uint32_t m, uint32_t k) { return qmm4c_q_bytes(m, k); }

}  // extern "C"
