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

// The no-allocation entry point's workspace (vkt_dispatch_static): a fixed array in the code object, one copy per
// device, held from the time the library's code is loaded until the process ends.  Host code never uses this name
// as an address: the runtime asks for the device address once (hipGetSymbolAddress, in runtime()) and passes that.
constexpr uint64_t kStaticScratchBytes = VKT_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr uint64_t kWorkspaceBytes = 32ull << 20;
// The widened-weights region of many-row int8 products is capped: larger weights run on the row-block kernels.
constexpr uint64_t kMaxWidenedBytes = 2ull << 30;

struct Runtime {
  int device = 0;
  hipDeviceProp_t props{};
  Machine machine;  // what the launchers see through vkt_dispatch
  hipStream_t stream = nullptr;
  std::mutex pool_mutex;  // lock order: pool, then stream (vkcore/src/lib.rs:33-50)
  std::mutex stream_mutex;
  std::unique_ptr<Pool<HipSource>> pool;
  std::atomic<uint64_t> dispatches{0};
  bool trace = false;
  uint64_t generation = 0;
  // The kernels' own memory, both pool allocations (so they show in vkt_memory_stats and go back with
  // vkt_empty_cache): the workspace of products split over workgroups, taken at the first vkt_dispatch, and the
  // widened-weights region, grown on demand.  Guarded by pool_mutex (the Machine fields also by stream_mutex).
  Allocation workspace_alloc{}, widened_alloc{};
  std::atomic<uint64_t> workspace_ready{0}, widened_ready{0};  // bytes of each that dispatches may count on
  // the smallest widened-weights size the pool has refused since the last vkt_empty_cache: such products run on the
  // row-block kernels without asking again (every failed attempt may trim the pool and wait for the device)
  std::atomic<uint64_t> widened_refused{UINT64_MAX};
  uint64_t static_scratch = 0;  // device address of `scratch` on this runtime's device

  // Makes sure the workspace exists and the widened-weights region holds `widened` bytes.  Called by vkt_dispatch
  // before it takes the stream: a new pool block is a hipMalloc, which may wait for the device.  Pool memory is
  // reused in stream order, so giving the old region back while queued kernels still read it is safe.
  bool ensure_kernel_memory(uint64_t widened, std::string* err) {
    std::lock_guard<std::mutex> lock(pool_mutex);
    if (workspace_alloc.size == 0) {
      Allocation a;
      if (!pool->alloc(kWorkspaceBytes, &a, err)) return false;
      std::lock_guard<std::mutex> stream_lock(stream_mutex);
      workspace_alloc = a;
      machine.workspace = a.address, machine.workspace_bytes = kWorkspaceBytes;
      workspace_ready.store(kWorkspaceBytes, std::memory_order_release);
    }
    if (widened > widened_alloc.size && widened <= kMaxWidenedBytes && widened < widened_refused.load(std::memory_order_relaxed)) {
      Allocation a;
      std::string ignored;  // (without memory for it the row-block kernels run)
      if (!pool->alloc(widened, &a, &ignored)) {
        widened_refused.store(widened, std::memory_order_relaxed);
      } else {
        std::lock_guard<std::mutex> stream_lock(stream_mutex);
        if (widened_alloc.size) pool->free(widened_alloc);
        widened_alloc = a;
        machine.scratch = a.address, machine.scratch_bytes = a.size;
        widened_ready.store(a.size, std::memory_order_release);
      }
    }
    return true;
  }
  // Gives the kernels' memory back to the pool (vkt_empty_cache).  Caller holds pool_mutex.
  void drop_kernel_memory() {
    std::lock_guard<std::mutex> stream_lock(stream_mutex);
    if (workspace_alloc.size) pool->free(workspace_alloc);
    if (widened_alloc.size) pool->free(widened_alloc);
    workspace_alloc = widened_alloc = Allocation{};
    machine.workspace = machine.workspace_bytes = machine.scratch = machine.scratch_bytes = 0;
    workspace_ready.store(0, std::memory_order_release), widened_ready.store(0, std::memory_order_release);
    widened_refused.store(UINT64_MAX, std::memory_order_relaxed);
  }

  ~Runtime() {
    if (stream) {
      (void)hipStreamSynchronize(stream);
    }
    pool.reset();
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
  // the device address of this device's copy of the fixed workspace (the array's name is not an address on the host)
  {
    void* at = nullptr;
    if ((e = hipGetSymbolAddress(&at, HIP_SYMBOL(scratch))) != hipSuccess || at == nullptr) {
      (void)hipGetLastError();
      *err = hip_message("hipGetSymbolAddress(scratch)", e);
      return nullptr;
    }
    rt->static_scratch = reinterpret_cast<uint64_t>(at);
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

// One dispatch as the launchers see it.
struct Call {
  const char* name;
  const char* rest;  // the name after the table entry's key (a dtype or size label), "" for exact names
  const uint32_t* spec;
  size_t nspec;
  uint32_t gz;
  const Machine& machine;
  hipStream_t stream;
  std::string* err;
  uint32_t spec_at(size_t i) const { return i < nspec ? spec[i] : 0u; }
};

int unknown_kernel(const Call& c) {
  *c.err = std::string("unknown kernel ") + c.name;
  return -1;
}

int call_qmm8(const Q8Params& p, const Call& c) {
  const int dt = dtype_of_suffix(c.rest);
  if (dt < 0) return unknown_kernel(c);
  // spec[0] is the reference's ROWS constant (0: tile path, 1..8: GEMV); the row count
  // that matters is p.m, so it is checked for consistency only.
  if (c.spec_at(0) != 0 && c.spec_at(0) != p.m) {
    *c.err = "qmm8: specialisation ROWS=" + std::to_string(c.spec_at(0)) + " does not match m=" + std::to_string(p.m);
    return -1;
  }
  return launch_qmm8(p, dt, c.spec_at(1), c.machine, c.stream, c.err);
}
int call_qmm4(const Q4Params& p, const Call& c) {
  const int dt = dtype_of_suffix(c.rest);
  if (dt != VKT_F32 && dt != VKT_BF16) return unknown_kernel(c);
  return launch_qmm4(p, dt, c.spec_at(0), c.spec_at(1), c.machine, c.stream, c.err);
}
int call_qmm4c(const Q4CParams& p, const Call& c) {
  const int dt = dtype_of_suffix(c.rest);
  if (dt != VKT_F32 && dt != VKT_BF16) return unknown_kernel(c);
  return launch_qmm4c(p, dt, c.spec_at(0), c.spec_at(1), c.spec_at(2), c.machine, c.stream, c.err);
}
int call_gemmcm(const GemmParams& p, const Call& c) {
  const int dt = dtype_of_suffix(c.rest);
  if (dt != VKT_BF16 && dt != VKT_F16) return unknown_kernel(c);
  return launch_gemm16(p, dt, c.spec_at(0), c.gz, c.spec_at(3), c.machine, c.stream, c.err);
}
int call_cast_strided(const StridedParams& p, const Call& c) {  // "cast_<src>_<dst>"
  const char* second = std::strchr(c.rest, '_');
  if (!second) return unknown_kernel(c);
  const int sdt = dtype_of_suffix(std::string(c.rest, second).c_str()), ddt = dtype_of_suffix(second + 1);
  if (sdt < 0 || ddt < 0 || sdt == ddt) return unknown_kernel(c);
  return launch_cast_strided(p, sdt, ddt, c.machine, c.stream, c.err);
}
int call_packvec(const Q4VecParams& p, const Call& c) { return launch_qmm4_packvec(p, c.stream, c.err); }
int call_qmm4c_pack(const Q4PackParams& p, const Call& c) { return launch_qmm4c_pack(p, c.spec_at(0), c.machine, c.stream, c.err); }
int call_move(const StridedParams& p, const Call& c) { return launch_move(p, c.rest, c.spec_at(0), c.spec_at(2), c.machine, c.stream, c.err); }
int call_copy8(const Copy8Params& p, const Call& c) { return launch_copy8(p, c.rest, c.spec_at(0), c.machine, c.stream, c.err); }
int call_cast_fp8(const CastParams& p, const Call& c) { return launch_cast_fp8(p, c.machine, c.stream, c.err); }
int call_quantize(const QuantParams& p, const Call& c) { return launch_quantize_affine(p, c.spec_at(0), false, c.machine, c.stream, c.err); }
int call_dequantize(const QuantParams& p, const Call& c) { return launch_quantize_affine(p, c.spec_at(0), true, c.machine, c.stream, c.err); }
int call_fake_quant(const QuantParams& p, const Call& c) { return launch_fake_quant(p, c.spec_at(0), c.spec_at(1), c.machine, c.stream, c.err); }
int call_aminmax(const MinMaxParams& p, const Call& c) { return launch_aminmax(p, c.machine, c.stream, c.err); }
int call_fp8_quant(const F8QuantParams& p, const Call& c) { return launch_fp8_quant(p, c.spec_at(0), c.machine, c.stream, c.err); }
int call_probe_read(const ProbeParams& p, const Call& c) { return launch_probe_read(p, c.spec_at(0), c.machine, c.stream, c.err); }
int call_probe_mfma(const ProbeParams& p, const Call& c) { return launch_probe_mfma(p, c.spec_at(0), c.machine, c.stream, c.err); }
int call_probe_delay(const ProbeParams& p, const Call& c) { return launch_probe_delay(p, c.stream, c.err); }
int call_fp8mm(const F8Params& p, const Call& c) { return launch_fp8mm(p, c.spec_at(0), c.machine, c.stream, c.err); }

// name -> parameter block type + launcher (the role of kernels.rs:72-140 KernelCache::get).  An entry ties a
// launcher to the one block type it takes, so a name cannot reach a launcher with another kernel's block.
struct KernelEntry {
  const char* key;
  bool prefix;  // the key is followed by a dtype / size label
  size_t param_bytes;
  int (*run)(const uint8_t* push, const Call& c);
};
template <class P, int (*F)(const P&, const Call&)>
int with_block(const uint8_t* push, const Call& c) {
  P p;
  std::memcpy(&p, push, sizeof(P));
  return F(p, c);
}
template <class P, int (*F)(const P&, const Call&)>
constexpr KernelEntry entry(const char* key, bool prefix) {
  return KernelEntry{key, prefix, sizeof(P), &with_block<P, F>};
}
// exact names first, so that "qmm4_packvec", "qmm4c_pack" and "cast_fp8" are not read as a prefix plus a label
const KernelEntry kKernels[] = {
    entry<Q4VecParams, call_packvec>("qmm4_packvec", false),
    entry<Q4PackParams, call_qmm4c_pack>("qmm4c_pack", false),
    entry<CastParams, call_cast_fp8>("cast_fp8", false),
    entry<QuantParams, call_quantize>("quantize_affine", false),
    entry<QuantParams, call_dequantize>("dequantize_affine", false),
    entry<QuantParams, call_fake_quant>("fake_quant", false),
    entry<MinMaxParams, call_aminmax>("aminmax", false),
    entry<F8QuantParams, call_fp8_quant>("fp8_quant", false),
    entry<F8Params, call_fp8mm>("fp8mm", false),
    entry<ProbeParams, call_probe_read>("probe_read", false),
    entry<ProbeParams, call_probe_mfma>("probe_mfma_f8", false),
    entry<ProbeParams, call_probe_delay>("probe_delay", false),
    entry<Q8Params, call_qmm8>("qmm8_", true),
    entry<Q4CParams, call_qmm4c>("qmm4c_", true),
    entry<Q4Params, call_qmm4>("qmm4_", true),
    entry<GemmParams, call_gemmcm>("gemmcm_", true),
    entry<StridedParams, call_move>("move_", true),
    entry<Copy8Params, call_copy8>("copy8_", true),
    entry<StridedParams, call_cast_strided>("cast_", true),
};

const KernelEntry* find_kernel(const char* name, const char** rest) {
  for (const KernelEntry& e : kKernels) {
    const size_t len = std::strlen(e.key);
    if (e.prefix ? std::strncmp(name, e.key, len) == 0 && name[len] != '\0' : std::strcmp(name, e.key) == 0) {
      *rest = name + (e.prefix ? len : std::strlen(name));
      return &e;
    }
  }
  return nullptr;
}

int dispatch_named(const Machine& machine, hipStream_t stream, const char* name, const uint32_t* spec, size_t nspec,
                   const uint8_t* push, size_t npush, uint32_t gz, std::string* err) {
  const char* rest = nullptr;
  const KernelEntry* e = find_kernel(name, &rest);
  if (!e) {
    *err = std::string("unknown kernel ") + name;
    return -1;
  }
  if (npush != e->param_bytes) {
    *err = std::string("kernel ") + name + " takes a parameter block of " + std::to_string(e->param_bytes) + " bytes, got " +
           std::to_string(npush);
    return -1;
  }
  const Call c{name, rest, spec, nspec, gz, machine, stream, err};
  return e->run(push, c);
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
  rt->drop_kernel_memory();  // (the next vkt_dispatch takes the workspace again)
  rt->pool->trim();
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

namespace {

// The common part of vkt_dispatch and vkt_dispatch_static: queue `name` on the runtime's stream against `machine`.
int queue_kernel(Runtime& rt, const Machine& machine, const char* name, const uint32_t* spec, size_t nspec,
                 const uint8_t* push, size_t npush, uint32_t gx, uint32_t gy, uint32_t gz) {
  std::string err;
  if (dispatch_named(machine, rt.stream, name, spec, nspec, push, npush, gz, &err) != 0) return fail(err);
  rt.dispatches.fetch_add(1, std::memory_order_relaxed);
  if (rt.trace) {
    // each kernel runs to completion before the next is queued, so a kernel that
    // faults is the last one printed (ffi.rs:135-142)
    std::fprintf(stderr, "[vkt] %s [", name);
    for (size_t i = 0; i < nspec; ++i) std::fprintf(stderr, i ? ", %u" : "%u", spec[i]);
    std::fprintf(stderr, "] grid %ux%ux%u\n", gx, gy, gz);
    std::fflush(stderr);
    hipError_t e = hipStreamSynchronize(rt.stream);
    if (e != hipSuccess) return fail(hip_message(name, e));
  }
  return 0;
}

int check_dispatch_arguments(const char* name, const uint8_t* push, size_t npush, uint32_t gx, uint32_t gy, uint32_t gz) {
  if (!name) return fail("kernel name is null");
  if (npush > 128) return fail("parameter blocks are limited to 128 bytes");
  if (npush != 0 && !push) return fail("parameter block is null");
  if (gx == 0 || gy == 0 || gz == 0) return fail("empty grid");
  return 0;
}

}  // namespace

int vkt_dispatch(const char* name, const uint32_t* spec, size_t nspec, const uint8_t* push, size_t npush, uint32_t gx,
                 uint32_t gy, uint32_t gz) {
  std::string err;
  auto rt = runtime(&err);
  if (!rt) return fail(err);
  if (check_dispatch_arguments(name, push, npush, gx, gy, gz) != 0) return -1;
  // The kernels' own memory comes from the pool, before the stream is taken (a new pool block is a hipMalloc, which
  // may wait for the device): the workspace at the first dispatch and after vkt_empty_cache; the widened-weights
  // region when a many-row int8 product first needs more of it than there is.
  uint64_t widened = 0;
  if (!std::strncmp(name, "qmm8_", 5) && npush == sizeof(Q8Params) && !((nspec > 1 ? spec[1] : 0u) >> 20 & 1)) {
    Q8Params p;
    std::memcpy(&p, push, sizeof(p));
    widened = q8_gemm_scratch_bytes(p, dtype_of_suffix(name + 5), rt->machine);
  }
  for (;;) {
    if ((rt->workspace_ready.load(std::memory_order_acquire) == 0 ||
         (widened > rt->widened_ready.load(std::memory_order_acquire) && widened < rt->widened_refused.load(std::memory_order_relaxed))) &&
        !rt->ensure_kernel_memory(widened, &err))
      return fail(err);
    std::lock_guard<std::mutex> lock(rt->stream_mutex);
    // (a vkt_empty_cache between the check above and this lock has taken the workspace away: take it again)
    if (rt->machine.workspace_bytes == 0) continue;
    return queue_kernel(*rt, rt->machine, name, spec, nspec, push, npush, gx, gy, gz);
  }
}

int vkt_dispatch_static(const char* name, const uint32_t* spec, size_t nspec, const uint8_t* push, size_t npush,
                        uint32_t gx, uint32_t gy, uint32_t gz) {
  auto rt = running();
  if (!rt) return fail("vkt_dispatch_static: the runtime is not running (start it with any other call, e.g. vkt_device_info)");
  if (check_dispatch_arguments(name, push, npush, gx, gy, gz) != 0) return -1;
  // the same launchers against a machine whose only kernel memory is the fixed array: a product that would need more
  // of it than kStaticScratchBytes is refused by its launcher (workspace_fixed), never shrunk or re-planned, and
  // nothing is widened into a second region
  Machine fixed;
  fixed.compute_units = rt->machine.compute_units;
  fixed.workspace = rt->static_scratch;
  fixed.workspace_bytes = kStaticScratchBytes;
  fixed.workspace_fixed = true;
  std::lock_guard<std::mutex> lock(rt->stream_mutex);
  return queue_kernel(*rt, fixed, name, spec, nspec, push, npush, gx, gy, gz);
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
  const char* rest = nullptr;
  return find_kernel(name, &rest) ? 64u : 0u;
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
  if (dst == src) return 0;  // a copy onto itself changes nothing (as on the CPU)
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
