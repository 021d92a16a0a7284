// Internals shared by the translation units of libacchip.  Not installed.
#pragma once
#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <atomic>
#include <condition_variable>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <set>
#include <memory>
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
void set_last_error(const std::string &message);
std::string last_error_text();
std::string compile_log_text();

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

// ---- tuning knobs -------------------------------------------------------------
// "scan.block=512,scan.rows=2,fold.unroll=8": overrides of the defaults that the generator and the drivers work
// with, for measurement sweeps.  The text is parsed ONCE into an immutable table -- the process's when it is first
// wanted (from ACC_HIP_TUNE in the environment) or set (acc_tuning_set), a context's when it is created or
// acc_context_set_tuning replaces it, an instance's when it is created -- so that nothing on the path of a driver call
// reads the environment.  A knob the generator reads becomes part of the source text and so of the cache key.
struct Tuning {
  std::vector<std::pair<std::string, int>> kv;      // sorted by name
  std::string text;
  int get(const char *name, int dflt) const;
  bool has(const char *name) const;
};
typedef std::shared_ptr<const Tuning> TuningPtr;
TuningPtr parse_tuning(const char *text);           // NULL or "": no overrides
TuningPtr default_tuning();                         // the process's table
void set_default_tuning(TuningPtr t);

// What the drivers look at on every call, resolved when an instance is created: plain integers.
#define ACC_DRIVER_KNOBS(X)                                                                                          \
  X(fold_blocks_per_cu, "fold.blocks_per_cu", 4)                                                                       \
  X(fold_rows_max, "fold.rows_max", 7)                                                                                 \
  X(fold_across, "fold.across", 2)                                                                                     \
  X(fold_across_min_piece, "fold.across_min_piece", 64)                                                                \
  X(foldseg_block_team_len, "foldseg.block_team_len", 16384)                                                           \
  X(foldseg_long_from, "foldseg.long_from", 8)                                                                         \
  X(foldseg_max_split, "foldseg.max_split", 4096)                                                                      \
  X(foldseg_oversub, "foldseg.oversub", 1 << 20)                                                                       \
  X(foldseg_giants, "foldseg.giants", 2)                                                                               \
  X(foldseg_giant_chunks, "foldseg.giant_chunks", 4)                                                                   \
  X(foldseg_sweep_per_cu, "foldseg.sweep_per_cu", 4)                                                                   \
  X(foldseg_row_team_below, "foldseg.row_team_below", 1024)                                                            \
  X(foldseg_wave_team_len, "foldseg.wave_team_len", 128)                                                               \
  X(map_oversub, "map.oversub", 1 << 20)                                                                               \
  X(permute_atomic_flush_max, "permute.atomic_flush_max", 1 << 16)                                                     \
  X(permute_fp_tables_from, "permute.fp_tables_from", 48)                                                              \
  X(permute_fp_tables_to, "permute.fp_tables_to", 6144)                                                                \
  X(permute_generic_lds, "permute.generic_lds", 1)                                                                     \
  X(permute_inline_fill, "permute.inline_fill", 1)                                                                     \
  X(permute_lds_bytes, "permute.lds_bytes", 160 * 1024)                                                                \
  X(permute_lock_copies_bytes, "permute.lock_copies_bytes", 40 * 1024)                                                 \
  X(permute_lock_lanes_per_target, "permute.lock_lanes_per_target", 32)                                                \
  X(permute_lock_lds_min_ratio, "permute.lock_lds_min_ratio", 4)                                                       \
  X(permute_lock_max_windows, "permute.lock_max_windows", 12)                                                          \
  X(permute_lock_table_mbytes, "permute.lock_table_mbytes", 64)                                                        \
  X(permute_max_blocks_per_cu, "permute.max_blocks_per_cu", 1)                                                         \
  X(permute_max_copies, "permute.max_copies", 16)                                                                      \
  X(permute_max_windows, "permute.max_windows", 32)                                                                    \
  X(permute_narrow, "permute.narrow", 1)                                                                               \
  X(permute_narrow_from, "permute.narrow_from", 8192)                                                                  \
  X(permute_windows_from, "permute.windows_from", 2)                                                                   \
  X(permute_xcd_row_kbytes, "permute.xcd_row_kbytes", 1024)                                                            \
  X(scan_small_below_kb, "scan.small_below_kb", 12288)                                                                 \
  X(stencil_half_strips, "stencil.half_strips", 1)                                                                     \
  X(map_tiled_min_w, "map.tiled_min_w", 33)                                                                          \
  X(map_tiled_min_h, "map.tiled_min_h", 10)                                                                          \
  X(stencil_thin_2d, "stencil.thin_2d", 36)                                                                          \
  X(stencil_thin_3d, "stencil.thin_3d", 16)                                                                          \
  X(stencil_narrow_max, "stencil.narrow_max", 2)                                                                       \
  X(stencil_stack, "stencil.stack", 0)                                                                                 \
  X(stencil_strips_per_cu, "stencil.strips_per_cu", 3)                                                                 \
  X(stencil_walk_min, "stencil.walk_min", 4)
struct Knobs {
#define ACC_KNOB_FIELD(field, name, dflt) int field = (dflt);
  ACC_DRIVER_KNOBS(ACC_KNOB_FIELD)
#undef ACC_KNOB_FIELD
  void resolve(const Tuning &t)
  {
#define ACC_KNOB_GET(field, name, dflt) field = t.get(name, (dflt));
    ACC_DRIVER_KNOBS(ACC_KNOB_GET)
#undef ACC_KNOB_GET
  }
};

// ---- compilation in the background ----------------------------------------------
// One run-time compilation handed to the worker pool (Compile.hs:620-660: forked threads bounded by the number of
// processors, the main thread carries on generating code and blocks at a kernel's first use, :451-457).  The job
// owns copies of everything the compiler reads, so the instance it was made for may go away meanwhile.
struct CompileJob {
  std::string target, source;
  std::vector<std::string> options;
  std::mutex mu;
  std::condition_variable cv;
  bool done = false;
  int rc = ACC_OK;
  std::string error, log;          // acc_last_error / acc_compile_log of the worker, for whoever waits
  const void *code = nullptr;      // owned by the kernel cache
  size_t size = 0;
  void run();                      // compile (through the cache) on the calling thread and mark done
  int wait();                      // block until done; the outcome, with error and log copied to the calling thread
};
// compilation in helper processes (compile_child.cpp): a pool thread attaches, and what it compiles from then on goes
// to its helper; compile_out_of_process is false where there is none (the caller then compiles in process)
void compile_child_attach();
void compile_child_detach();
bool compile_out_of_process(const std::string &target, const char *source, const std::vector<std::string> &options,
                            std::vector<char> *code, std::string *log, int *rc);
// hiprtc on the calling thread (cache.cpp): the code object, the log in the thread's compile log
int compile_in_process(const std::string &target, const char *source, const std::vector<std::string> &options, std::vector<char> *code);
bool compile_submit(const std::shared_ptr<CompileJob> &job);     // false: the pool has been drained, nothing was queued
void compile_drain();
int compile_pool_threads();

// ---- staged transfers (transfer.cpp) ----------------------------------------------
class Stager;
void stager_destroy(acc_context ctx);
bool wants_staging(acc_context ctx, const void *host, size_t bytes);
// the upload is handed to the copy engine on the stager's stream `*on`, *done is recorded behind it
int staged_upload(acc_context ctx, void *dev, const void *host, size_t bytes, hipEvent_t *done, hipStream_t *on);
int staged_upload_wait(acc_context ctx);
int staged_download(acc_context ctx, void *host, const void *dev, size_t bytes);     // returns with the data in `host`

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
// Behind them, in the same block: words that say something else than "a wait ran out" -- a kernel of a segmented fold
// met a very long segment (execute.cpp, launch_segmented).  An instance takes the next word in turn; two instances
// that share one may each take the other's hint for its own, which costs them a variant they did not need.
enum { HINT_WORDS = 1024 };

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

  // the tuning table instances created in this context take (set under `mu`)
  acc::TuningPtr tuning;
  acc::TuningPtr tuning_now()
  {
    std::lock_guard<std::mutex> lock(mu);
    return tuning;
  }
  bool dump_exec = false;      // ACC_HIP_DEBUG=dump-exec was in the environment when the context was created

  // large copies from and to pageable host memory go through pinned buffers of the context's own (transfer.cpp)
  acc::Stager *stager = nullptr;
  int copy_helpers = 3;                  // threads that copy beside the caller (knob copy.threads, the caller included)
  size_t copy_staged_from = 4u << 20;    // bytes from which a pageable copy is staged (knob copy.staged_from_kb; the largest size_t with copy.staged=0: never)

  // kernels report here that a bounded wait ran out (see StatusWord); NULL if the block could not be set up
  volatile uint32_t *status_host = nullptr;
  std::atomic<unsigned> next_hint{0};
  uint64_t status_dev = 0;

  // Streams and events that were given back while nothing was pending on them wait here for the next request
  // (the reservoir of Execute/Stream.hs:118-140 and the event table of Execute/Event.hs:63-85), under `mu`.
  std::vector<hipStream_t> spare_streams;
  std::vector<hipEvent_t> spare_events[2];          // [0] without timing, [1] with
  std::set<hipEvent_t> timed_events;                // the events of acc_event_create that record times (an event does not say)
  static constexpr size_t SPARE_MAX = 64;

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
  // a borrower could not leave a SCRATCH_LOCKS / SCRATCH_CARRY block as it found it: cleared before it is lent again
  void scratch_mark_dirty(const acc::ScratchRef &ref);
  // free every block that is not lent and whose last use has completed; returns the bytes given back
  size_t scratch_trim();
  size_t scratch_bytes();
  // ACC_ERR_STUCK (once) if a kernel has reported a wait that ran out since the last call
  int check_status(const char *who);
};
