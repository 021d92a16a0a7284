// The one translation unit of libacchip with device code of its own, built by hipcc for gfx950: a file-scope array
// in device memory that serves as the scan's tile-descriptor block for callers that must not allocate
// (acc_exec_scan_noalloc), and the small kernel that clears it.
//
// The array's name is a host-side stand-in for the symbol, not a device address: its address on a device is asked
// for once per device, with that device current, and kept; everything that touches the memory afterwards -- kernel
// arguments, the clearing kernel -- goes through that pointer.  Every device the library runs on holds its own copy
// of the array (ACC_NOALLOC_SCRATCH_BYTES) until the process ends.
#include <hip/hip_runtime.h>

#include <mutex>

#include "acc_internal.hpp"

static __device__ __align__(256) unsigned char scratch[ACC_NOALLOC_SCRATCH_BYTES];

namespace {

// zero `words` 8-byte words from p on (a kernel, not a memset node, so that a caller may capture the launch)
__global__ void __launch_bounds__(256) acc_noalloc_clear(unsigned long long *p, size_t words)
{
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += (size_t)gridDim.x * 256) p[i] = 0ull;
}

constexpr int MAX_DEVICES = 64;

struct DeviceScratch {
  std::mutex mu;
  bool asked = false;
  hipError_t status = hipErrorNotInitialized;
  void *ptr = nullptr;        // the array's address on this device
  uint32_t epoch = 0;         // tag of the last scan that used it (acc::SCRATCH_SCAN: stale tags read as "not yet")
};
DeviceScratch g_dev[MAX_DEVICES];

}  // namespace

namespace acc {

// Once per device, with that device current (acc_context_create calls it): ask for the array's address there.
int noalloc_setup(int device)
{
  if (device < 0 || device >= MAX_DEVICES) return ACC_OK;      // such a device has no scratch: the entry point says so
  DeviceScratch &d = g_dev[device];
  std::lock_guard<std::mutex> lock(d.mu);
  if (d.asked) return ACC_OK;
  void *p = nullptr;
  d.status = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  d.ptr = d.status == hipSuccess ? p : nullptr;
  d.asked = true;
  if (d.status != hipSuccess) (void)hipGetLastError();
  return ACC_OK;
}

// The descriptor block of one scan launch on `device` (current): its address and the launch's tag.  Nothing is
// allocated; the block is shared by every call on the device, so calls that overlap there race.
int noalloc_scan_state(int device, size_t bytes, hipStream_t stream, void **base, uint32_t *epoch)
{
  if (device < 0 || device >= MAX_DEVICES) return fail(ACC_ERR_UNSUPPORTED, "acc_exec_scan_noalloc: no scratch for device %d", device);
  DeviceScratch &d = g_dev[device];
  std::lock_guard<std::mutex> lock(d.mu);
  if (!d.asked || d.status != hipSuccess || !d.ptr)
    return fail(ACC_ERR_HIP, "acc_exec_scan_noalloc: the scratch array has no address on device %d (%s)", device,
                d.asked ? hipGetErrorString(d.status) : "no context was created on it");
  if (bytes > (size_t)ACC_NOALLOC_SCRATCH_BYTES)
    return fail(ACC_ERR_INVALID, "acc_exec_scan_noalloc: %zu bytes of tile descriptors needed, the scratch array holds %d", bytes,
                (int)ACC_NOALLOC_SCRATCH_BYTES);
  if (d.epoch + 1 >= (1u << 30)) {            // descriptor tags are 30 bits wide: start over from a clean block
    hipLaunchKernelGGL(acc_noalloc_clear, dim3(64), dim3(256), 0, stream, static_cast<unsigned long long *>(d.ptr),
                       (size_t)ACC_NOALLOC_SCRATCH_BYTES / 8);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "acc_noalloc_clear");
    d.epoch = 0;
  }
  *epoch = ++d.epoch;
  *base = d.ptr;
  return ACC_OK;
}

}  // namespace acc
