// A stand-in for the HIP runtime, in the process and without a device, for ONE purpose: building libacchip's host
// code under ThreadSanitizer and driving it from many threads (driver.cpp).  Memory is host memory, streams and
// events are small heap objects, a launch does nothing.  hiprtc is the real one (it needs no device).  The two units
// of the library that carry device code of their own (noalloc.hip, guard.hip) are not part of this build; what the
// host code calls in them is defined at the end of this file.
//
// Test infrastructure only: nothing of the product links this.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../accelerate-cuda_amd/csrc/acc_internal.hpp"

namespace {
std::atomic<long> g_launches{0};
struct Stream { int id; };
struct Event { std::atomic<int> recorded{0}; };
struct Module { const void *image; };
struct Function { char name[64]; };
}  // namespace

extern "C" {

long mock_hip_launches(void) { return g_launches.load(); }

hipError_t hipInit(unsigned) { return hipSuccess; }
hipError_t hipGetDeviceCount(int *n) { *n = 1; return hipSuccess; }
hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
hipError_t hipGetLastError(void) { return hipSuccess; }
const char *hipGetErrorString(hipError_t) { return "mock error"; }
hipError_t hipDeviceSynchronize(void) { return hipSuccess; }

hipError_t hipGetDevicePropertiesR0600(hipDeviceProp_t *p, int d)
{
  if (d != 0) return hipErrorInvalidDevice;
  std::memset(p, 0, sizeof(*p));
  std::strcpy(p->name, "mock MI355X");
  std::strcpy(p->gcnArchName, "gfx950:sramecc+:xnack-");
  p->multiProcessorCount = 256;
  p->warpSize = 64;
  p->maxThreadsPerBlock = 1024;
  p->clockRate = 2400000;
  p->sharedMemPerBlock = 160 * 1024;
  p->maxSharedMemoryPerMultiProcessor = 160 * 1024;
  p->l2CacheSize = 4 << 20;
  p->totalGlobalMem = size_t(1) << 36;
  p->regsPerBlock = 65536;
  p->maxThreadsPerMultiProcessor = 2048;
  return hipSuccess;
}

hipError_t hipMalloc(void **p, size_t n) { *p = std::malloc(n ? n : 1); return *p ? hipSuccess : hipErrorOutOfMemory; }
hipError_t hipFree(void *p) { std::free(p); return hipSuccess; }
hipError_t hipHostMalloc(void **p, size_t n, unsigned) { *p = std::calloc(1, n ? n : 1); return *p ? hipSuccess : hipErrorOutOfMemory; }
hipError_t hipHostFree(void *p) { std::free(p); return hipSuccess; }
hipError_t hipPointerGetAttributes(hipPointerAttribute_t *, const void *) { return hipErrorInvalidValue; }    // every host address is pageable here
hipError_t hipHostGetDevicePointer(void **d, void *h, unsigned) { *d = h; return hipSuccess; }
hipError_t hipMemGetInfo(size_t *f, size_t *t) { *f = size_t(1) << 35; *t = size_t(1) << 36; return hipSuccess; }
// (copies and fills are not carried out: two threads of the driver may name the same "device" buffers, as two
// streams of a real program may, and what the device would do with them is not the host code's business)
hipError_t hipMemcpy(void *, const void *, size_t, hipMemcpyKind) { return hipSuccess; }
hipError_t hipMemcpyAsync(void *, const void *, size_t, hipMemcpyKind, hipStream_t) { return hipSuccess; }
hipError_t hipMemsetAsync(void *, int, size_t, hipStream_t) { return hipSuccess; }
hipError_t hipMemsetD32Async(hipDeviceptr_t, int, size_t, hipStream_t) { return hipSuccess; }

hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { *s = reinterpret_cast<hipStream_t>(new Stream{0}); return hipSuccess; }
hipError_t hipStreamDestroy(hipStream_t s) { delete reinterpret_cast<Stream *>(s); return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipStreamQuery(hipStream_t) { return hipSuccess; }
hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *e) { *e = reinterpret_cast<hipEvent_t>(new Event()); return hipSuccess; }
hipError_t hipEventCreateWithFlags(hipEvent_t *e, unsigned) { return hipEventCreate(e); }
hipError_t hipEventDestroy(hipEvent_t e) { delete reinterpret_cast<Event *>(e); return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t e, hipStream_t) { reinterpret_cast<Event *>(e)->recorded.store(1); return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventQuery(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) { *ms = 0.001f; return hipSuccess; }

hipError_t hipModuleLoadData(hipModule_t *m, const void *image) { *m = reinterpret_cast<hipModule_t>(new Module{image}); return hipSuccess; }
hipError_t hipModuleUnload(hipModule_t m) { delete reinterpret_cast<Module *>(m); return hipSuccess; }
hipError_t hipModuleGetFunction(hipFunction_t *f, hipModule_t, const char *name)
{
  Function *fn = new Function();          // (leaked: a function handle lives as long as its module in the real runtime)
  std::strncpy(fn->name, name, sizeof(fn->name) - 1);
  *f = reinterpret_cast<hipFunction_t>(fn);
  return hipSuccess;
}
const char *hipKernelNameRef(const hipFunction_t f) { return reinterpret_cast<const Function *>(f)->name; }
hipError_t hipFuncGetAttribute(int *v, hipFunction_attribute a, hipFunction_t)
{
  *v = a == HIP_FUNC_ATTRIBUTE_NUM_REGS ? 96 : 0;
  return hipSuccess;
}
hipError_t hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(int *n, hipFunction_t, int block, size_t lds)
{
  const int by_lds = lds ? static_cast<int>((160 * 1024) / lds) : 8;
  *n = std::max(1, std::min({8, 2048 / std::max(64, block), by_lds}));
  return hipSuccess;
}
// The one kernel that does something here: a segmented fold's look at its segment lengths (<entry>_probe) finds a very
// long segment once the driver says so -- it sets the word whose address is its argument number `g_probe_arg`, as the
// kernel would -- so that the instance's change to its other variants happens among the threads that launch it.
static std::atomic<int> g_probe_arg{-1};
static std::atomic<long> g_sweeps{0};
hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, hipStream_t,
                                 void **params, void **)
{
  g_launches.fetch_add(1);
  const char *name = reinterpret_cast<const Function *>(f)->name;
  const size_t len = std::strlen(name);
  const int at = g_probe_arg.load();
  if (len > 6 && std::strcmp(name + len - 6, "_sweep") == 0) g_sweeps.fetch_add(1);
  if (at >= 0 && params && len > 6 && std::strcmp(name + len - 6, "_probe") == 0) {
    unsigned int *word = *reinterpret_cast<unsigned int **>(params[at]);
    __atomic_store_n(word, 1u, __ATOMIC_RELAXED);
  }
  return hipSuccess;
}
void mock_hip_probe_finds(int argument) { g_probe_arg.store(argument); }
long mock_hip_sweeps(void) { return g_sweeps.load(); }

}  // extern "C"

// ---- what the host code calls in noalloc.hip and guard.hip -------------------------------------------------------

struct acc_guard_s {
  acc_context ctx = nullptr;
  unsigned int words[2] = {1u, 0u};
};

namespace acc {

int noalloc_setup(int) { return ACC_OK; }

int noalloc_scan_state(int, size_t bytes, hipStream_t, void **base, uint32_t *epoch)
{
  static unsigned char block[ACC_NOALLOC_SCRATCH_BYTES];
  static std::mutex mu;
  static uint32_t tag = 0;
  if (bytes > sizeof(block)) return fail(ACC_ERR_INVALID, "mock: too many tiles");
  std::lock_guard<std::mutex> lock(mu);
  *base = block;
  *epoch = ++tag;
  return ACC_OK;
}

int guarded_copy(uint64_t, uint64_t, size_t, uint64_t, hipStream_t)
{
  g_launches.fetch_add(1);
  return ACC_OK;
}

}  // namespace acc

extern "C" {

int acc_guard_create(acc_context ctx, acc_guard *out)
{
  acc_guard g = new acc_guard_s();
  g->ctx = ctx;
  *out = g;
  return ACC_OK;
}

int acc_guard_destroy(acc_guard g)
{
  if (!g) return ACC_OK;
  {
    std::lock_guard<std::mutex> lock(g->ctx->mu);
    const uint64_t at = reinterpret_cast<uint64_t>(g->words);
    for (auto it = g->ctx->guards.begin(); it != g->ctx->guards.end();) {
      if (it->second == at) {
        it = g->ctx->guards.erase(it);
        g->ctx->n_guards.fetch_sub(1, std::memory_order_release);
      } else {
        ++it;
      }
    }
  }
  delete g;
  return ACC_OK;
}

int acc_guard_reset(acc_guard, acc_stream) { return ACC_OK; }
int acc_guard_latch(acc_guard, const acc_array *, acc_stream) { return ACC_OK; }
int acc_guard_read(acc_guard g, acc_stream, int32_t *alive, int64_t *count)
{
  if (alive) *alive = 0;
  if (count) *count = 0;
  return g->ctx->check_status("acc_guard_read");
}

int acc_stream_set_guard(acc_context ctx, acc_stream stream, acc_guard g)
{
  hipStream_t st = static_cast<hipStream_t>(stream);
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto it = ctx->guards.find(st);
  if (!g) {
    if (it != ctx->guards.end()) {
      ctx->guards.erase(it);
      ctx->n_guards.fetch_sub(1, std::memory_order_release);
    }
    return ACC_OK;
  }
  if (it == ctx->guards.end()) {
    ctx->guards[st] = reinterpret_cast<uint64_t>(g->words);
    ctx->n_guards.fetch_add(1, std::memory_order_release);
  } else {
    it->second = reinterpret_cast<uint64_t>(g->words);
  }
  return ACC_OK;
}

}  // extern "C"
