// Internals shared by the translation units of libacchip.  Not installed.
#pragma once
#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/acc_hip.h"

#define ACC_HIP_VERSION "0.1.0"

// bytes of the file-scope device array behind acc_exec_scan_noalloc: a 256-byte header and one 128-byte tile
// descriptor for each of ACC_NOALLOC_MAX_TILES tiles (noalloc.hip)
#define ACC_NOALLOC_SCRATCH_BYTES (256 + ACC_NOALLOC_MAX_TILES * 128)

namespace acc {

// thread-local message of the last failure; returns `code` so that call
// sites read `return fail(ACC_ERR_INVALID, "...")`
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t e, const char *what);
void set_compile_log(const std::string &log);

#define ACC_HIP_TRY(expr)                                  \
  do {                                                     \
    hipError_t _e = (expr);                                \
    if (_e != hipSuccess) return ::acc::fail_hip(_e, #expr); \
  } while (0)

#define ACC_TRY(expr)            \
  do {                           \
    int _rc = (expr);            \
    if (_rc != ACC_OK) return _rc; \
  } while (0)

// the scan's descriptor block for callers that must not allocate (noalloc.hip)
int noalloc_setup(int device);
int noalloc_scan_state(int device, size_t bytes, hipStream_t stream, void **base, uint32_t *epoch);

// embedded device headers (embed.cpp)
struct EmbeddedHeader { const char *name; const char *begin; const char *end; };
const std::vector<EmbeddedHeader> &embedded_headers();
std::string embedded_text(const char *name);

// A block of device memory lent to one skeleton launch (tile descriptors,
// block partials, tickets).  Blocks are reused when the borrowing stream is
// the same (stream order makes that safe) or the event recorded at release
// has completed.
enum ScratchProtocol {
  SCRATCH_FOLD = 0,   // contents are don't-care: every launch writes what it reads (fold partials, permute tables)
  SCRATCH_LOCKS = 2,  // all zero between uses: every launch leaves it as it found it
  SCRATCH_CARRY = 4,  // the same contract, for the carries of the counting permute (a pool of their own, so that the
                      // lock blocks stay what acc_context_debug_poke_lock takes them for)
  SCRATCH_SCAN = 1,   // tile descriptors (behind a 256-byte header nothing uses): they carry `epoch`, so stale
                      // ones read as "not yet published"
  SCRATCH_FLAGS = 3   // 64-bit words {epoch, payload}: every launch tags what it writes with its `epoch`,
                      // anything older reads as "not yet"
};

struct ScratchBlock {
  void *ptr = nullptr;
  size_t bytes = 0;
  int protocol = SCRATCH_FOLD;
  hipStream_t stream = nullptr;
  hipEvent_t done = nullptr;
  bool busy = false;
  bool recorded = false;   // `done` was recorded at the last release
  bool dirty = false;      // SCRATCH_LOCKS / SCRATCH_CARRY: a launch may have left it non-zero: cleared again before it is lent
  uint32_t epoch = 0;
};

// What a borrower holds of a block: copies taken under the pool's lock (the pool's vector may move meanwhile).
// `epoch` is the tag of this use for the SCRATCH_SCAN / SCRATCH_FLAGS protocols (the pool starts a block over from
// zeroes before its tags run out).
struct ScratchRef {
  int index = -1;
  void *ptr = nullptr;
  size_t bytes = 0;
  uint32_t epoch = 0;
};

// Words of a context's status block (pinned host memory that kernels write, the host reads at synchronisation
// points): non-zero = a kernel's bounded wait ran out since the block was last read.
enum StatusWord { STATUS_SCAN_LOOKBACK = 0, STATUS_FOLD_COLLECT = 1, STATUS_PERMUTE_LOCK = 2, STATUS_WORDS = 16 };

// big single-pass scans on different streams of one device are kept from overlapping (runtime.cpp)
// device-to-device copy of `bytes` bytes that does nothing when the guard word at `guard` is zero (guard.hip)
int guarded_copy(uint64_t dst, uint64_t src, size_t bytes, uint64_t guard, hipStream_t stream);

int scan_order_before(int device, hipStream_t stream);    // ACC_OK: the caller launches, then calls scan_order_after
void scan_order_after(int device);
void scan_order_forget(int device, hipStream_t stream);

}  // namespace acc

struct acc_context_s {
  int device = 0;
  hipDeviceProp_t props;
  std::string arch;          // "gfx950"
  std::mutex mu;
  std::vector<acc::ScratchBlock> scratch;
  // Completion events are only needed to hand a block from one stream to
  // another.  While a single stream has used the pool, stream order alone
  // makes reuse safe and no events are recorded.
  bool scratch_any_stream = false;
  bool scratch_multi_stream = false;
  hipStream_t scratch_first_stream = nullptr;

  // kernels report here that a bounded wait ran out (see StatusWord); NULL if the block could not be set up
  volatile uint32_t *status_host = nullptr;
  uint64_t status_dev = 0;

  // streams with a loop's guard set (acc_stream_set_guard) and the address of its `alive` word
  std::map<hipStream_t, uint64_t> guards;
  std::atomic<int> n_guards{0};
  uint64_t guard_of(hipStream_t stream)
  {
    if (n_guards.load(std::memory_order_acquire) == 0) return 0;
    std::lock_guard<std::mutex> lock(mu);
    auto it = guards.find(stream);
    return it == guards.end() ? 0 : it->second;
  }

  int make_current() const;
  // zero-initialised when first allocated; contents persist between uses and
  // follow the block's protocol
  int scratch_acquire(size_t bytes, hipStream_t stream, int protocol, acc::ScratchRef *out);
  void scratch_release(const acc::ScratchRef &ref, hipStream_t stream);
  // free every block that is not lent and whose last use has completed; returns the bytes given back
  size_t scratch_trim();
  size_t scratch_bytes();
  // ACC_ERR_STUCK (once) if a kernel has reported a wait that ran out since the last call
  int check_status(const char *who);
};
