// Driver layer of libacchip: devices, contexts, memory, transfers, streams,
// events, modules, occupancy and raw launches over libamdhip64.
//
// It stands where accelerate-cuda reaches the `cuda` package:
//   State.hs:127-132, Context.hs:55-111      initialise / create / destroy
//   Array/Remote.hs:63-79,191                mallocArray / free / getMemInfo
//   Array/Prim.hs:189-391                    peek / poke / copy [Async]
//   Execute/Stream.hs, Execute/Event.hs      stream and event handling
//   Compile.hs:453-465,505,534               loadData / getFun / requires
//   Execute.hs:975-978                       launchKernel
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "acc_internal.hpp"

namespace acc {

static thread_local std::string g_last_error;
static thread_local std::string g_compile_log;

int fail(int code, const char *fmt, ...)
{
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int fail_hip(hipError_t e, const char *what)
{
  // the one error a caller is expected to recover from (Array/Remote.hs:63-67)
  const int code = (e == hipErrorOutOfMemory) ? ACC_ERR_OOM : ACC_ERR_HIP;
  (void)hipGetLastError();  // do not let a sticky error leak into the next call
  return fail(code, "%s: %s (%d)", what, hipGetErrorString(e), static_cast<int>(e));
}

void set_compile_log(const std::string &log) { g_compile_log = log; }
void set_last_error(const std::string &message) { g_last_error = message; }
std::string last_error_text() { return g_last_error; }
std::string compile_log_text() { return g_compile_log; }

// ---- tuning knobs ------------------------------------------------------------

int Tuning::get(const char *name, int dflt) const
{
  auto it = std::lower_bound(kv.begin(), kv.end(), name,
                             [](const std::pair<std::string, int> &e, const char *n) { return e.first.compare(n) < 0; });
  return (it != kv.end() && it->first == name) ? it->second : dflt;
}

bool Tuning::has(const char *name) const
{
  auto it = std::lower_bound(kv.begin(), kv.end(), name,
                             [](const std::pair<std::string, int> &e, const char *n) { return e.first.compare(n) < 0; });
  return it != kv.end() && it->first == name;
}

TuningPtr parse_tuning(const char *text)
{
  auto t = std::make_shared<Tuning>();
  t->text = text ? text : "";
  const std::string &all = t->text;
  size_t pos = 0;
  while (pos < all.size()) {
    size_t end = all.find(',', pos);
    if (end == std::string::npos) end = all.size();
    const size_t eq = all.find('=', pos);
    if (eq != std::string::npos && eq < end && eq > pos) {
      std::string name = all.substr(pos, eq - pos);
      while (!name.empty() && name.front() == ' ') name.erase(name.begin());
      while (!name.empty() && name.back() == ' ') name.pop_back();
      // the first setting of a name wins, as it did when the text was searched from the left
      bool seen = false;
      for (const auto &e : t->kv) seen = seen || e.first == name;
      if (!seen && !name.empty()) t->kv.emplace_back(name, std::atoi(all.c_str() + eq + 1));
    }
    pos = end + 1;
  }
  std::sort(t->kv.begin(), t->kv.end());
  return t;
}

static std::mutex g_tuning_mu;
static TuningPtr g_tuning;

TuningPtr default_tuning()
{
  std::lock_guard<std::mutex> lock(g_tuning_mu);
  if (!g_tuning) g_tuning = parse_tuning(std::getenv("ACC_HIP_TUNE"));     // once, when first wanted
  return g_tuning;
}

void set_default_tuning(TuningPtr t)
{
  std::lock_guard<std::mutex> lock(g_tuning_mu);
  g_tuning = std::move(t);
}

}  // namespace acc

using acc::fail;

int acc_context_s::make_current() const
{
  ACC_HIP_TRY(hipSetDevice(device));
  return ACC_OK;
}

int acc_context_s::scratch_acquire(size_t bytes, hipStream_t stream, int protocol, acc::ScratchRef *out)
{
  std::lock_guard<std::mutex> lock(mu);
  if (!scratch_any_stream) {
    scratch_any_stream = true;
    scratch_first_stream = stream;
  } else if (!scratch_multi_stream && stream != scratch_first_stream) {
    // a second stream shows up: settle everything enqueued so far once, and
    // track completion with events from here on
    ACC_HIP_TRY(hipDeviceSynchronize());
    scratch_multi_stream = true;
  }
  int pick = -1;
  for (size_t i = 0; i < scratch.size(); ++i) {
    acc::ScratchBlock &b = scratch[i];
    if (b.busy || b.bytes < bytes || b.protocol != protocol) continue;
    bool reusable = (b.stream == stream) || !b.recorded;
    if (!reusable) reusable = (hipEventQuery(b.done) == hipSuccess);
    if (reusable && (pick < 0 || b.bytes < scratch[pick].bytes)) pick = static_cast<int>(i);
  }
  if (pick < 0) {
    acc::ScratchBlock b;
    b.bytes = (bytes + 4095) & ~size_t(4095);
    ACC_HIP_TRY(hipMalloc(&b.ptr, b.bytes));
    // into an entry that a trim has emptied, if there is one (it keeps its event)
    for (size_t i = 0; i < scratch.size() && pick < 0; ++i)
      if (!scratch[i].ptr && !scratch[i].busy) pick = static_cast<int>(i);
    if (pick >= 0) {
      b.done = scratch[pick].done;
    } else {
      hipError_t e = hipEventCreateWithFlags(&b.done, hipEventDisableTiming);
      if (e != hipSuccess) { (void)hipFree(b.ptr); return acc::fail_hip(e, "hipEventCreateWithFlags"); }
    }
    b.protocol = protocol;
    b.dirty = true;         // cleared below, on the stream that first uses it (not meant to be captured into a graph)
    if (pick >= 0) {
      scratch[pick] = b;
    } else {
      scratch.push_back(b);
      pick = static_cast<int>(scratch.size()) - 1;
    }
  }
  acc::ScratchBlock &b = scratch[pick];
  // tags: the scan's are 30 bits wide, the tagged words' 32
  const bool tags_out = (protocol == acc::SCRATCH_SCAN && b.epoch + 1 >= (1u << 30)) || (protocol == acc::SCRATCH_FLAGS && b.epoch == 0xFFFFFFFFu);
  if (b.dirty || tags_out) {
    hipError_t e = hipMemsetAsync(b.ptr, 0, b.bytes, stream);
    if (e != hipSuccess) return acc::fail_hip(e, "hipMemsetAsync(scratch)");
    b.dirty = false;
    b.epoch = 0;
  }
  if (protocol == acc::SCRATCH_SCAN || protocol == acc::SCRATCH_FLAGS) ++b.epoch;
  b.busy = true;
  b.stream = stream;
  out->index = pick;
  out->ptr = b.ptr;
  out->bytes = b.bytes;
  out->epoch = b.epoch;
  return ACC_OK;
}

void acc_context_s::scratch_release(const acc::ScratchRef &ref, hipStream_t stream)
{
  if (ref.index < 0) return;
  std::lock_guard<std::mutex> lock(mu);
  acc::ScratchBlock &b = scratch[ref.index];
  b.recorded = false;
  if (scratch_multi_stream) b.recorded = (hipEventRecord(b.done, stream) == hipSuccess);
  b.stream = stream;
  b.busy = false;
}

void acc_context_s::scratch_mark_dirty(const acc::ScratchRef &ref)
{
  if (ref.index < 0) return;
  std::lock_guard<std::mutex> lock(mu);
  scratch[ref.index].dirty = true;
}

size_t acc_context_s::scratch_bytes()
{
  std::lock_guard<std::mutex> lock(mu);
  size_t total = 0;
  for (const acc::ScratchBlock &b : scratch) total += b.ptr ? b.bytes : 0;
  return total;
}

// Blocks keep their place in the vector (borrowers hold indices): a freed one stays as an empty entry that matches
// no request and is filled again by the next allocation that finds no block.
size_t acc_context_s::scratch_trim()
{
  std::lock_guard<std::mutex> lock(mu);
  size_t freed = 0;
  for (acc::ScratchBlock &b : scratch) {
    if (b.busy || !b.ptr) continue;
    if (hipFree(b.ptr) != hipSuccess) { (void)hipGetLastError(); continue; }      // hipFree waits for the device itself
    freed += b.bytes;
    b.ptr = nullptr;
    b.bytes = 0;
    b.epoch = 0;
    b.recorded = false;
  }
  // empty entries at the end can go
  while (!scratch.empty() && !scratch.back().ptr && !scratch.back().busy) {
    if (scratch.back().done) (void)hipEventDestroy(scratch.back().done);
    scratch.pop_back();
  }
  return freed;
}

int acc_context_s::check_status(const char *who)
{
  if (!status_host) return ACC_OK;
  uint32_t seen[acc::STATUS_WORDS];
  bool any = false;
  for (int k = 0; k < acc::STATUS_WORDS; ++k) {
    seen[k] = status_host[k];
    any = any || seen[k] != 0;
  }
  if (!any) return ACC_OK;
  {
    std::lock_guard<std::mutex> lock(mu);
    for (int k = 0; k < acc::STATUS_WORDS; ++k) status_host[k] = 0;
    // a lock that never opened is still set: every lock block is cleared before it is lent again
    for (acc::ScratchBlock &b : scratch)
      if (b.protocol == acc::SCRATCH_LOCKS || b.protocol == acc::SCRATCH_CARRY) b.dirty = true;
  }
  return fail(ACC_ERR_STUCK, "%s: a kernel gave up waiting (%s%s%s): results of the work enqueued since the last successful synchronisation are not valid",
              who, seen[acc::STATUS_SCAN_LOOKBACK] ? "scan look-back " : "", seen[acc::STATUS_FOLD_COLLECT] ? "fold partial results " : "",
              seen[acc::STATUS_PERMUTE_LOCK] ? "permute lock" : "");
}

namespace acc {

// Two single-pass scans whose grids exceed what is resident at once must not share the device: each compute die
// hands out the workgroups of a launch in order, but the dies do so independently of one another, so tiles of scan A
// could fill one die waiting for an A tile that another die, full of waiting tiles of scan B, has no room for (and
// the other way round).  Within a process such scans are therefore chained, per device: a scan on another stream
// than the last one waits for an event recorded on that stream just then (everything enqueued there so far, the
// earlier scan included).  Scans that follow one another on one stream -- the common case -- cost nothing.
// scan_order_before takes the device's lock and scan_order_after gives it back, so that the launch itself lies
// between them: a second thread must not record its event before the first one's scan is enqueued.
struct ScanOrder {
  std::mutex mu;
  hipEvent_t ev = nullptr;
  hipStream_t last = nullptr;
  bool have_last = false;     // `last` is the stream of the most recent big scan (and still exists)
  bool ev_pending = false;    // that stream is gone; `ev` was recorded on it before it went
};
static ScanOrder g_scan_order[64];

int scan_order_before(int device, hipStream_t stream)
{
  if (device < 0 || device >= 64) return ACC_OK;
  ScanOrder &o = g_scan_order[device];
  o.mu.lock();
  hipError_t e = hipSuccess;
  if (o.have_last && o.last != stream) {
    if (!o.ev) e = hipEventCreateWithFlags(&o.ev, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventRecord(o.ev, o.last);
    if (e == hipSuccess) e = hipStreamWaitEvent(stream, o.ev, 0);
  } else if (!o.have_last && o.ev_pending) {
    e = hipStreamWaitEvent(stream, o.ev, 0);
  }
  if (e != hipSuccess) {
    o.mu.unlock();
    return fail_hip(e, "ordering of scans on different streams");
  }
  o.have_last = true;
  o.last = stream;
  o.ev_pending = false;
  return ACC_OK;
}

void scan_order_after(int device)
{
  if (device < 0 || device >= 64) return;
  g_scan_order[device].mu.unlock();
}

// a stream is about to be destroyed: what it still holds of a big scan is remembered by an event
void scan_order_forget(int device, hipStream_t stream)
{
  if (device < 0 || device >= 64) return;
  ScanOrder &o = g_scan_order[device];
  std::lock_guard<std::mutex> lock(o.mu);
  if (!o.have_last || o.last != stream) return;
  o.have_last = false;
  o.last = nullptr;
  hipError_t e = hipSuccess;
  if (!o.ev) e = hipEventCreateWithFlags(&o.ev, hipEventDisableTiming);
  if (e == hipSuccess) e = hipEventRecord(o.ev, stream);
  o.ev_pending = (e == hipSuccess);
  if (e != hipSuccess) { (void)hipGetLastError(); (void)hipStreamSynchronize(stream); }
}

}  // namespace acc

extern "C" {

const char *acc_last_error(void) { return acc::g_last_error.c_str(); }
const char *acc_compile_log(void) { return acc::g_compile_log.c_str(); }
const char *acc_version(void) { return ACC_HIP_VERSION; }

int acc_init(void)
{
  ACC_HIP_TRY(hipInit(0));
  return ACC_OK;
}

int acc_device_count(int *count)
{
  if (!count) return fail(ACC_ERR_INVALID, "acc_device_count: NULL argument");
  *count = 0;
  ACC_HIP_TRY(hipGetDeviceCount(count));
  return ACC_OK;
}

static void fill_props(const hipDeviceProp_t &p, acc_device_props *out)
{
  std::memset(out, 0, sizeof(*out));
  std::snprintf(out->name, sizeof(out->name), "%s", p.name);
  std::snprintf(out->arch, sizeof(out->arch), "%.63s", p.gcnArchName);
  out->compute_units = p.multiProcessorCount;
  out->wavefront_size = p.warpSize;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  out->clock_khz = p.clockRate;
  out->lds_per_block = static_cast<int64_t>(p.sharedMemPerBlock);
  out->lds_per_cu = static_cast<int64_t>(p.maxSharedMemoryPerMultiProcessor);
  out->l2_bytes = p.l2CacheSize;
  out->total_mem = static_cast<int64_t>(p.totalGlobalMem);
  out->regs_per_block = p.regsPerBlock;
  out->max_threads_per_cu = p.maxThreadsPerMultiProcessor;
}

int acc_device_get_props(int device, acc_device_props *out)
{
  if (!out) return fail(ACC_ERR_INVALID, "acc_device_get_props: NULL argument");
  hipDeviceProp_t p;
  ACC_HIP_TRY(hipGetDeviceProperties(&p, device));
  fill_props(p, out);
  return ACC_OK;
}

int acc_context_create(int device, acc_context *out)
{
  if (!out) return fail(ACC_ERR_INVALID, "acc_context_create: NULL argument");
  *out = nullptr;
  int n = 0;
  ACC_HIP_TRY(hipGetDeviceCount(&n));
  if (device < 0 || device >= n) return fail(ACC_ERR_NOT_FOUND, "acc_context_create: no device %d (%d present)", device, n);
  acc_context_s *ctx = new acc_context_s();
  ctx->device = device;
  hipError_t e = hipGetDeviceProperties(&ctx->props, device);
  if (e == hipSuccess) e = hipSetDevice(device);
  if (e != hipSuccess) { delete ctx; return acc::fail_hip(e, "acc_context_create"); }
  (void)acc::noalloc_setup(device);      // the address of the library's own device array on this device, once
  {
    // the status block: host memory the device can write (only ever written when a kernel's bounded wait runs out)
    void *hp = nullptr, *dp = nullptr;
    if (hipHostMalloc(&hp, (acc::STATUS_WORDS + acc::HINT_WORDS) * sizeof(uint32_t), hipHostMallocMapped) == hipSuccess &&
        hipHostGetDevicePointer(&dp, hp, 0) == hipSuccess) {
      std::memset(hp, 0, (acc::STATUS_WORDS + acc::HINT_WORDS) * sizeof(uint32_t));
      ctx->status_host = static_cast<volatile uint32_t *>(hp);
      ctx->status_dev = reinterpret_cast<uint64_t>(dp);
    } else {
      (void)hipGetLastError();
      if (hp) (void)hipHostFree(hp);
    }
  }
  ctx->tuning = acc::default_tuning();
  ctx->copy_helpers = std::max(1, ctx->tuning->get("copy.threads", 4)) - 1;
  ctx->copy_staged_from = ctx->tuning->get("copy.staged", 1) ? (size_t)std::max(1, ctx->tuning->get("copy.staged_from_kb", 4096)) << 10 : ~size_t(0);
  {
    const char *dbg = std::getenv("ACC_HIP_DEBUG");      // looked at here, never on the path of a launch
    ctx->dump_exec = dbg && std::strstr(dbg, "dump-exec");
  }
  ctx->arch = ctx->props.gcnArchName;
  const size_t colon = ctx->arch.find(':');
  if (colon != std::string::npos) ctx->arch.resize(colon);
  *out = ctx;
  return ACC_OK;
}

int acc_context_destroy(acc_context ctx)
{
  if (!ctx) return ACC_OK;
  (void)hipSetDevice(ctx->device);
  (void)hipDeviceSynchronize();
  acc::stager_destroy(ctx);
  for (hipStream_t st : ctx->spare_streams) (void)hipStreamDestroy(st);
  for (auto &pool : ctx->spare_events)
    for (hipEvent_t ev : pool) (void)hipEventDestroy(ev);
  for (acc::ScratchBlock &b : ctx->scratch) {
    if (b.done) (void)hipEventDestroy(b.done);
    if (b.ptr) (void)hipFree(b.ptr);
  }
  if (ctx->status_host) (void)hipHostFree(const_cast<uint32_t *>(ctx->status_host));
  delete ctx;
  return ACC_OK;
}

int acc_tuning_set(const char *text)
{
  // NULL: what ACC_HIP_TUNE holds in the environment now
  acc::set_default_tuning(acc::parse_tuning(text ? text : std::getenv("ACC_HIP_TUNE")));
  return ACC_OK;
}

const char *acc_tuning_text(void)
{
  static thread_local std::string text;
  text = acc::default_tuning()->text;
  return text.c_str();
}

int acc_context_set_tuning(acc_context ctx, const char *text)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_context_set_tuning: NULL context");
  acc::TuningPtr t = text ? acc::parse_tuning(text) : acc::default_tuning();
  std::lock_guard<std::mutex> lock(ctx->mu);
  ctx->tuning = t;
  return ACC_OK;
}

int acc_context_device(acc_context ctx, int *device)
{
  if (!ctx || !device) return fail(ACC_ERR_INVALID, "acc_context_device: NULL argument");
  *device = ctx->device;
  return ACC_OK;
}

int acc_context_sync(acc_context ctx)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_context_sync: NULL context");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipDeviceSynchronize());
  return ctx->check_status("acc_context_sync");
}

int acc_context_trim(acc_context ctx, size_t *freed_bytes)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_context_trim: NULL context");
  ACC_TRY(ctx->make_current());
  const size_t freed = ctx->scratch_trim();
  if (freed_bytes) *freed_bytes = freed;
  return ACC_OK;
}

int acc_context_debug_poke_lock(acc_context ctx, size_t word, uint32_t value)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_context_debug_poke_lock: NULL context");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipDeviceSynchronize());
  void *at = nullptr;
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    const acc::ScratchBlock *found = nullptr;
    for (const acc::ScratchBlock &b : ctx->scratch)
      if (b.protocol == acc::SCRATCH_LOCKS && b.ptr && !b.busy) found = &b;
    if (!found) return fail(ACC_ERR_NOT_FOUND, "acc_context_debug_poke_lock: the context holds no lock block");
    // (the locks start 256 bytes into their block)
    if (256 + (word + 1) * 4 > found->bytes) return fail(ACC_ERR_INVALID, "acc_context_debug_poke_lock: word %zu lies outside the block", word);
    at = static_cast<char *>(found->ptr) + 256 + word * 4;
  }
  ACC_HIP_TRY(hipMemcpy(at, &value, 4, hipMemcpyHostToDevice));
  return ACC_OK;
}

int acc_context_scratch_bytes(acc_context ctx, size_t *bytes)
{
  if (!ctx || !bytes) return fail(ACC_ERR_INVALID, "acc_context_scratch_bytes: NULL argument");
  *bytes = ctx->scratch_bytes();
  return ACC_OK;
}

int acc_malloc(acc_context ctx, size_t bytes, acc_devptr *out)
{
  if (!ctx || !out) return fail(ACC_ERR_INVALID, "acc_malloc: NULL argument");
  *out = 0;
  ACC_TRY(ctx->make_current());
  void *p = nullptr;
  // a zero-sized array still needs a distinct, valid pointer (Array/Prim.hs:150-157)
  ACC_HIP_TRY(hipMalloc(&p, bytes ? bytes : 1));
  *out = reinterpret_cast<acc_devptr>(p);
  return ACC_OK;
}

int acc_free(acc_context ctx, acc_devptr p)
{
  if (!p) return ACC_OK;
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_free: NULL context");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipFree(reinterpret_cast<void *>(p)));
  return ACC_OK;
}

int acc_mem_info(acc_context ctx, size_t *free_bytes, size_t *total_bytes)
{
  if (!ctx || !free_bytes || !total_bytes) return fail(ACC_ERR_INVALID, "acc_mem_info: NULL argument");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
  return ACC_OK;
}

int acc_host_alloc(acc_context ctx, size_t bytes, void **out)
{
  if (!ctx || !out) return fail(ACC_ERR_INVALID, "acc_host_alloc: NULL argument");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault));
  return ACC_OK;
}

int acc_host_free(acc_context ctx, void *p)
{
  if (!p) return ACC_OK;
  // (page-locked memory belongs to the process, not to a device: a buffer may outlive the context it was asked
  // from, and is then given back with no context)
  if (ctx) ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipHostFree(p));
  return ACC_OK;
}

static int copy(acc_context ctx, void *dst, const void *src, size_t bytes, hipMemcpyKind kind, hipStream_t s, bool async)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "memcpy: NULL context");
  if (bytes == 0) return ACC_OK;
  if (!dst || !src) return fail(ACC_ERR_INVALID, "memcpy: NULL pointer");
  ACC_TRY(ctx->make_current());
  if (async) {
    ACC_HIP_TRY(hipMemcpyAsync(dst, src, bytes, kind, s));
  } else {
    ACC_HIP_TRY(hipMemcpy(dst, src, bytes, kind));
  }
  return ACC_OK;
}

// The blocking copies keep the ordering of a copy on the default stream -- behind the work queued there before, done
// when the call returns -- also where they are staged through the context's pinned buffers on a stream of its own.
int acc_memcpy_h2d(acc_context c, acc_devptr d, const void *s, size_t n)
{
  if (c && d && s && n && acc::wants_staging(c, s, n)) {
    ACC_TRY(c->make_current());
    ACC_HIP_TRY(hipStreamSynchronize(nullptr));
    ACC_TRY(acc::staged_upload(c, reinterpret_cast<void *>(d), s, n, nullptr, nullptr));
    return acc::staged_upload_wait(c);
  }
  return copy(c, reinterpret_cast<void *>(d), s, n, hipMemcpyHostToDevice, nullptr, false);
}
int acc_memcpy_d2h(acc_context c, void *d, acc_devptr s, size_t n)
{
  // (a blocking copy to the host is where most callers first look at a result: a kernel's report is returned here too)
  if (c && d && s && n && acc::wants_staging(c, d, n)) {
    ACC_TRY(c->make_current());
    ACC_HIP_TRY(hipStreamSynchronize(nullptr));
    ACC_TRY(acc::staged_download(c, d, reinterpret_cast<void *>(s), n));
  } else {
    ACC_TRY(copy(c, d, reinterpret_cast<void *>(s), n, hipMemcpyDeviceToHost, nullptr, false));
  }
  return c->check_status("acc_memcpy_d2h");
}
int acc_memcpy_d2d(acc_context c, acc_devptr d, acc_devptr s, size_t n) { return copy(c, reinterpret_cast<void *>(d), reinterpret_cast<void *>(s), n, hipMemcpyDeviceToDevice, nullptr, false); }
int acc_memcpy_h2d_async(acc_context c, acc_devptr d, const void *s, size_t n, acc_stream st) { return copy(c, reinterpret_cast<void *>(d), s, n, hipMemcpyHostToDevice, static_cast<hipStream_t>(st), true); }
int acc_memcpy_d2h_async(acc_context c, void *d, acc_devptr s, size_t n, acc_stream st) { return copy(c, d, reinterpret_cast<void *>(s), n, hipMemcpyDeviceToHost, static_cast<hipStream_t>(st), true); }
int acc_memcpy_d2d_async(acc_context c, acc_devptr d, acc_devptr s, size_t n, acc_stream st) { return copy(c, reinterpret_cast<void *>(d), reinterpret_cast<void *>(s), n, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(st), true); }

int acc_memset32_async(acc_context ctx, acc_devptr dst, uint32_t value, size_t count, acc_stream s)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_memset32_async: NULL context");
  if (count == 0) return ACC_OK;
  if (!dst) return fail(ACC_ERR_INVALID, "acc_memset32_async: NULL pointer");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(dst), static_cast<int>(value), count, static_cast<hipStream_t>(s)));
  return ACC_OK;
}

int acc_stream_create(acc_context ctx, acc_stream *out)
{
  if (!ctx || !out) return fail(ACC_ERR_INVALID, "acc_stream_create: NULL argument");
  ACC_TRY(ctx->make_current());
  {
    // one that was given back idle, if there is one (Execute/Stream.hs:66-74 looks into its reservoir first)
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!ctx->spare_streams.empty()) {
      *out = ctx->spare_streams.back();
      ctx->spare_streams.pop_back();
      return ACC_OK;
    }
  }
  hipStream_t s;
  // default priority on purpose; non-blocking w.r.t. the NULL stream as CUDA.Stream.create [] is not
  ACC_HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *out = s;
  return ACC_OK;
}

int acc_stream_destroy(acc_context ctx, acc_stream s)
{
  if (!s) return ACC_OK;
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_stream_destroy: NULL context");
  ACC_TRY(ctx->make_current());
  acc::scan_order_forget(ctx->device, static_cast<hipStream_t>(s));
  {
    // a guard set on the stream goes with it: a later stream commonly gets the same handle value
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (ctx->guards.erase(static_cast<hipStream_t>(s)) != 0) ctx->n_guards.fetch_sub(1, std::memory_order_release);
  }
  // A stream with nothing pending is kept for the next acc_stream_create (Execute/Stream.hs:118-140 returns a
  // stream to the reservoir once its work is done); one that still has work is destroyed, which lets that work
  // finish and frees the stream behind it.
  if (hipStreamQuery(static_cast<hipStream_t>(s)) == hipSuccess) {
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (ctx->spare_streams.size() < acc_context_s::SPARE_MAX) {
      ctx->spare_streams.push_back(static_cast<hipStream_t>(s));
      return ACC_OK;
    }
  } else {
    (void)hipGetLastError();                      // hipErrorNotReady is no error of this call
  }
  ACC_HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(s)));
  return ACC_OK;
}

int acc_stream_sync(acc_context ctx, acc_stream s)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_stream_sync: NULL context");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(s)));
  return ctx->check_status("acc_stream_sync");
}

int acc_stream_wait_event(acc_context ctx, acc_stream s, acc_event e)
{
  if (!ctx || !e) return fail(ACC_ERR_INVALID, "acc_stream_wait_event: NULL argument");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(s), static_cast<hipEvent_t>(e), 0));
  return ACC_OK;
}

int acc_event_create(acc_context ctx, int enable_timing, acc_event *out)
{
  if (!ctx || !out) return fail(ACC_ERR_INVALID, "acc_event_create: NULL argument");
  ACC_TRY(ctx->make_current());
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto &pool = ctx->spare_events[enable_timing ? 1 : 0];
    if (!pool.empty()) {
      *out = pool.back();
      pool.pop_back();
      return ACC_OK;
    }
  }
  hipEvent_t e;
  ACC_HIP_TRY(hipEventCreateWithFlags(&e, enable_timing ? hipEventDefault : hipEventDisableTiming));
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (enable_timing) ctx->timed_events.insert(e);
  }
  *out = e;
  return ACC_OK;
}

int acc_event_destroy(acc_context ctx, acc_event e)
{
  if (!e) return ACC_OK;
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_event_destroy: NULL context");
  ACC_TRY(ctx->make_current());
  // An event that is not waiting for anything (never recorded, or what it was recorded behind has completed) is
  // kept for the next acc_event_create of its kind (Execute/Event.hs:63-85 keeps a table of such events).
  const hipError_t q = hipEventQuery(static_cast<hipEvent_t>(e));
  if (q != hipSuccess) (void)hipGetLastError();
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    const bool timed = ctx->timed_events.count(static_cast<hipEvent_t>(e)) != 0;
    auto &pool = ctx->spare_events[timed ? 1 : 0];
    if (q == hipSuccess && pool.size() < acc_context_s::SPARE_MAX) {
      pool.push_back(static_cast<hipEvent_t>(e));
      return ACC_OK;
    }
    if (timed) ctx->timed_events.erase(static_cast<hipEvent_t>(e));
  }
  ACC_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(e)));
  return ACC_OK;
}

int acc_event_record(acc_context ctx, acc_event e, acc_stream s)
{
  if (!ctx || !e) return fail(ACC_ERR_INVALID, "acc_event_record: NULL argument");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(e), static_cast<hipStream_t>(s)));
  return ACC_OK;
}

int acc_event_sync(acc_context ctx, acc_event e)
{
  if (!ctx || !e) return fail(ACC_ERR_INVALID, "acc_event_sync: NULL argument");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(e)));
  return ctx->check_status("acc_event_sync");
}

int acc_event_query(acc_context ctx, acc_event e, int *done)
{
  if (!ctx || !e || !done) return fail(ACC_ERR_INVALID, "acc_event_query: NULL argument");
  ACC_TRY(ctx->make_current());
  hipError_t r = hipEventQuery(static_cast<hipEvent_t>(e));
  if (r == hipSuccess) { *done = 1; return ACC_OK; }
  if (r == hipErrorNotReady) { *done = 0; (void)hipGetLastError(); return ACC_OK; }
  return acc::fail_hip(r, "hipEventQuery");
}

int acc_event_elapsed_ms(acc_context ctx, acc_event start, acc_event stop, float *ms)
{
  if (!ctx || !start || !stop || !ms) return fail(ACC_ERR_INVALID, "acc_event_elapsed_ms: NULL argument");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return ACC_OK;
}

int acc_module_load(acc_context ctx, const void *code, size_t code_size, acc_module *out)
{
  if (!ctx || !code || !code_size || !out) return fail(ACC_ERR_INVALID, "acc_module_load: NULL argument");
  ACC_TRY(ctx->make_current());
  hipModule_t m;
  ACC_HIP_TRY(hipModuleLoadData(&m, code));
  *out = m;
  return ACC_OK;
}

int acc_module_unload(acc_context ctx, acc_module m)
{
  if (!m) return ACC_OK;
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_module_unload: NULL context");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipModuleUnload(static_cast<hipModule_t>(m)));
  return ACC_OK;
}

int acc_module_get_function(acc_context ctx, acc_module m, const char *entry, acc_function *out)
{
  if (!ctx || !m || !entry || !out) return fail(ACC_ERR_INVALID, "acc_module_get_function: NULL argument");
  ACC_TRY(ctx->make_current());
  hipFunction_t f;
  hipError_t e = hipModuleGetFunction(&f, static_cast<hipModule_t>(m), entry);
  if (e == hipErrorNotFound) { (void)hipGetLastError(); return fail(ACC_ERR_NOT_FOUND, "no kernel entry '%s' in module", entry); }
  if (e != hipSuccess) return acc::fail_hip(e, "hipModuleGetFunction");
  *out = f;
  return ACC_OK;
}

int acc_function_attr(acc_context ctx, acc_function f, int which, int *value)
{
  if (!ctx || !f || !value) return fail(ACC_ERR_INVALID, "acc_function_attr: NULL argument");
  hipFunction_attribute a;
  switch (which) {
    case ACC_FUNC_NUM_REGS: a = HIP_FUNC_ATTRIBUTE_NUM_REGS; break;
    case ACC_FUNC_SHARED_SIZE_BYTES: a = HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES; break;
    case ACC_FUNC_CONST_SIZE_BYTES: a = HIP_FUNC_ATTRIBUTE_CONST_SIZE_BYTES; break;
    case ACC_FUNC_LOCAL_SIZE_BYTES: a = HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES; break;
    case ACC_FUNC_MAX_THREADS: a = HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK; break;
    default: return fail(ACC_ERR_INVALID, "acc_function_attr: unknown attribute %d", which);
  }
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipFuncGetAttribute(value, a, static_cast<hipFunction_t>(f)));
  return ACC_OK;
}

int acc_occupancy(acc_context ctx, acc_function f, int block, size_t dyn_lds, int *blocks_per_cu)
{
  if (!ctx || !f || !blocks_per_cu || block <= 0) return fail(ACC_ERR_INVALID, "acc_occupancy: bad argument");
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(blocks_per_cu, static_cast<hipFunction_t>(f), block, dyn_lds));
  return ACC_OK;
}

int acc_launch(acc_context ctx, acc_function f, uint32_t grid, uint32_t block, uint32_t dyn_lds, acc_stream s, void **args)
{
  if (!ctx || !f) return fail(ACC_ERR_INVALID, "acc_launch: NULL argument");
  if (grid == 0 || block == 0 || block > static_cast<uint32_t>(ctx->props.maxThreadsPerBlock))
    return fail(ACC_ERR_INVALID, "acc_launch: bad launch shape grid=%u block=%u", grid, block);
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipModuleLaunchKernel(static_cast<hipFunction_t>(f), grid, 1, 1, block, 1, 1, dyn_lds,
                                    static_cast<hipStream_t>(s), args, nullptr));
  return ACC_OK;
}

int64_t acc_launch_grid(int64_t n, int64_t per_block, int64_t cus, int64_t blocks_per_cu)
{
  if (per_block < 1) per_block = 1;
  int64_t need = (n + per_block - 1) / per_block;
  if (need < 1) need = 1;
  int64_t cap = cus * blocks_per_cu;
  if (cap < 1) cap = 1;
  return need < cap ? need : cap;
}

}  // extern "C"
