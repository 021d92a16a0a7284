// The guard of an array-level loop: awhile (Execute.hs:236-244) without a host round trip per iteration.
//
// Two words in device memory, `alive` and `count`.  The skeletons of the loop's predicate and body are built with
// ACC_FLAG_GUARDED: their kernels load `alive` on entry and return when it is zero.  Between predicate and body a
// one-lane kernel, acc_guard_latch, folds the predicate's Bool into `alive` and counts the iterations that are really
// taken.  The host enqueues several iterations, then reads both words; the iterations enqueued past the loop's end
// have done nothing.  The kernels here are built by hipcc with the library (they take no generated code).
#include <hip/hip_runtime.h>

#include "acc_internal.hpp"

using acc::fail;

struct acc_guard_s {
  acc_context ctx = nullptr;
  unsigned int *dev = nullptr;       // [0] alive, [1] count
  unsigned int *host = nullptr;      // pinned, two words: where acc_guard_read has them copied
};

namespace {

__global__ void acc_guard_reset_kernel(unsigned int *g)
{
  if (threadIdx.x == 0) {
    g[0] = 1u;
    g[1] = 0u;
  }
}

// alive := alive && pred;  count += alive
__global__ void acc_guard_latch_kernel(unsigned int *g, const unsigned char *pred)
{
  if (threadIdx.x == 0) {
    const unsigned int alive = (g[0] != 0u && *pred != 0) ? 1u : 0u;
    g[0] = alive;
    g[1] += alive;
  }
}

// bytes from src to dst unless the guard is down: 16 bytes a lane where both are aligned, single bytes at the ragged end
__global__ void __launch_bounds__(256) acc_guarded_copy_kernel(unsigned char *dst, const unsigned char *src, size_t bytes, const unsigned int *guard)
{
  if (*guard == 0u) return;
  const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, step = (size_t)gridDim.x * 256;
  size_t done = 0;
  if ((((uintptr_t)dst | (uintptr_t)src) & 15u) == 0) {
    const size_t vecs = bytes / 16;
    const uint4 *s4 = reinterpret_cast<const uint4 *>(src);
    uint4 *d4 = reinterpret_cast<uint4 *>(dst);
    for (size_t i = tid; i < vecs; i += step) d4[i] = s4[i];
    done = vecs * 16;
  }
  for (size_t i = done + tid; i < bytes; i += step) dst[i] = src[i];
}

}  // namespace

namespace acc {

int guarded_copy(uint64_t dst, uint64_t src, size_t bytes, uint64_t guard, hipStream_t stream)
{
  if (bytes == 0) return ACC_OK;
  const size_t lanes = (bytes + 15) / 16;
  const unsigned grid = static_cast<unsigned>(std::min<size_t>((lanes + 255) / 256, 2048));
  hipLaunchKernelGGL(acc_guarded_copy_kernel, dim3(grid), dim3(256), 0, stream, reinterpret_cast<unsigned char *>(dst),
                     reinterpret_cast<const unsigned char *>(src), bytes, reinterpret_cast<const unsigned int *>(guard));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "guarded copy");
  return ACC_OK;
}

}  // namespace acc

extern "C" {

int acc_guard_create(acc_context ctx, acc_guard *out)
{
  if (!ctx || !out) return fail(ACC_ERR_INVALID, "acc_guard_create: NULL argument");
  *out = nullptr;
  ACC_TRY(ctx->make_current());
  acc_guard g = new acc_guard_s();
  g->ctx = ctx;
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&g->dev), 256);
  if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&g->host), 2 * sizeof(unsigned int), hipHostMallocDefault);
  const unsigned int init[2] = {1u, 0u};
  if (e == hipSuccess) e = hipMemcpy(g->dev, init, sizeof(init), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    if (g->dev) (void)hipFree(g->dev);
    if (g->host) (void)hipHostFree(g->host);
    delete g;
    return acc::fail_hip(e, "acc_guard_create");
  }
  *out = g;
  return ACC_OK;
}

int acc_guard_destroy(acc_guard g)
{
  if (!g) return ACC_OK;
  (void)g->ctx->make_current();
  {
    // no stream keeps pointing at memory that is about to go
    std::lock_guard<std::mutex> lock(g->ctx->mu);
    const uint64_t at = reinterpret_cast<uint64_t>(g->dev);
    for (auto it = g->ctx->guards.begin(); it != g->ctx->guards.end();) {
      if (it->second == at) {
        it = g->ctx->guards.erase(it);
        g->ctx->n_guards.fetch_sub(1, std::memory_order_release);
      } else {
        ++it;
      }
    }
  }
  (void)hipFree(g->dev);          // waits for the device
  (void)hipHostFree(g->host);
  delete g;
  return ACC_OK;
}

int acc_guard_reset(acc_guard g, acc_stream stream)
{
  if (!g) return fail(ACC_ERR_INVALID, "acc_guard_reset: NULL guard");
  ACC_TRY(g->ctx->make_current());
  hipLaunchKernelGGL(acc_guard_reset_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), g->dev);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return acc::fail_hip(e, "acc_guard_reset");
  return ACC_OK;
}

int acc_guard_latch(acc_guard g, const acc_array *pred, acc_stream stream)
{
  if (!g || !pred) return fail(ACC_ERR_INVALID, "acc_guard_latch: NULL argument");
  if (pred->rank != 0 || pred->ncomp != 1 || !pred->ptr[0])
    return fail(ACC_ERR_INVALID, "acc_guard_latch: the predicate's result is a rank-0 array of Bool (one byte)");
  ACC_TRY(g->ctx->make_current());
  hipLaunchKernelGGL(acc_guard_latch_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), g->dev,
                     reinterpret_cast<const unsigned char *>(pred->ptr[0]));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return acc::fail_hip(e, "acc_guard_latch");
  return ACC_OK;
}

int acc_guard_read(acc_guard g, acc_stream stream, int32_t *alive, int64_t *count)
{
  if (!g) return fail(ACC_ERR_INVALID, "acc_guard_read: NULL guard");
  ACC_TRY(g->ctx->make_current());
  hipStream_t st = static_cast<hipStream_t>(stream);
  ACC_HIP_TRY(hipMemcpyAsync(g->host, g->dev, 2 * sizeof(unsigned int), hipMemcpyDeviceToHost, st));
  ACC_HIP_TRY(hipStreamSynchronize(st));
  if (alive) *alive = static_cast<int32_t>(g->host[0]);
  if (count) *count = static_cast<int64_t>(g->host[1]);
  return g->ctx->check_status("acc_guard_read");
}

int acc_stream_set_guard(acc_context ctx, acc_stream stream, acc_guard g)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_stream_set_guard: NULL context");
  if (g && g->ctx != ctx) return fail(ACC_ERR_INVALID, "acc_stream_set_guard: the guard belongs to another context");
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
    ctx->guards[st] = reinterpret_cast<uint64_t>(g->dev);
    ctx->n_guards.fetch_add(1, std::memory_order_release);
  } else {
    it->second = reinterpret_cast<uint64_t>(g->dev);
  }
  return ACC_OK;
}

}  // extern "C"
