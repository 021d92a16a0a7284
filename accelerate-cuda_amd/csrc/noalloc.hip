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

// The tag of the next scan: one more than the last one's, kept in the first word of the array's header and read from
// there by the scan kernel (a launch recorded into a graph carries the same arguments on every replay, so the tag
// cannot be one of them: this kernel is recorded in front of the scan and counts on the device).  When the 30 bits a
// descriptor has for its tag run out, the descriptors are cleared and the count starts again -- here too, not on the
// host, and by stores of a kernel, not by a memset node.
__global__ void __launch_bounds__(256) acc_noalloc_next_tag(unsigned int *header, unsigned long long *desc, size_t words)
{
  __shared__ unsigned int next;
  if (threadIdx.x == 0) next = header[0] + 1u;
  __syncthreads();
  const unsigned int tag = next;
  if (tag >= (1u << 30)) {
    for (size_t i = threadIdx.x; i < words; i += 256) desc[i] = 0ull;
    if (threadIdx.x == 0) header[0] = 1u;
  } else if (threadIdx.x == 0) {
    header[0] = tag;
  }
}

constexpr int MAX_DEVICES = 64;

struct DeviceScratch {
  std::mutex mu;
  bool asked = false;
  hipError_t status = hipErrorNotInitialized;
  void *ptr = nullptr;        // the array's address on this device
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
  // the launch's tag is counted on the device, by a kernel in front of the scan on the same stream (so that a graph
  // that records both gets a fresh tag at every replay); the scan is told to look there by a tag of 0
  hipLaunchKernelGGL(acc_noalloc_next_tag, dim3(1), dim3(256), 0, stream, static_cast<unsigned int *>(d.ptr),
                     reinterpret_cast<unsigned long long *>(static_cast<char *>(d.ptr) + 256), ((size_t)ACC_NOALLOC_SCRATCH_BYTES - 256) / 8);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "acc_noalloc_next_tag");
  *epoch = 0;
  *base = d.ptr;
  return ACC_OK;
}

}  // namespace acc
