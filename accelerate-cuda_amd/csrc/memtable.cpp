// Memory table: host array identity -> device block, a nursery of freed blocks
// keyed by size, and least-recently-used eviction (write-back to the host copy
// unless that copy is authoritative).  One table belongs to one context, hence
// one device; every entry point takes the table's lock.
#include <algorithm>
#include <unordered_map>

#include "acc_internal.hpp"

using namespace acc;

namespace {

enum Status {
  CLEAN,      // device == host
  DIRTY,      // device holds the only current copy
  EVICTED,    // host holds the only copy; no device block
  PENDING,    // frozen, not uploaded yet; device block may or may not exist
  UNMANAGED   // the caller's device memory
};

// the end of the work queued on one stream when an array was last released there
struct Use {
  hipStream_t stream = nullptr;
  hipEvent_t done = nullptr;
};

struct Entry {
  void *host = nullptr;
  uint64_t bytes = 0, rounded = 0;
  void *dev = nullptr;
  Status status = CLEAN;
  bool frozen = false;
  int pins = 0;
  uint64_t tick = 0;           // last acquire
  std::vector<Use> uses;       // one per stream with work that may still touch the block
  hipStream_t upload_stream = nullptr;
  hipEvent_t uploaded = nullptr;   // set while the upload may still be running: other streams wait for it
};

// a block waiting for reuse, with the work that may still touch it
struct FreeBlock {
  void *dev = nullptr;
  std::vector<Use> uses;
};

uint64_t round_up(uint64_t bytes)
{
  uint64_t b = bytes ? bytes : 1;
  return (b + ACC_MEMTABLE_GRANULE - 1) / ACC_MEMTABLE_GRANULE * ACC_MEMTABLE_GRANULE;
}

}  // namespace

struct acc_memtable_s {
  acc_context ctx = nullptr;
  uint64_t budget = 0;
  std::mutex mu;
  std::unordered_map<uint64_t, Entry> table;
  std::multimap<uint64_t, FreeBlock> nursery;  // rounded size -> free block
  std::vector<hipEvent_t> spare_events;
  uint64_t clock = 0;
  acc_memtable_stats st{};

  uint64_t held() const { return st.resident_bytes + st.nursery_bytes; }

  int event(hipEvent_t *out)
  {
    if (!spare_events.empty()) { *out = spare_events.back(); spare_events.pop_back(); return ACC_OK; }
    ACC_HIP_TRY(hipEventCreateWithFlags(out, hipEventDisableTiming));
    return ACC_OK;
  }

  // wait for everything in `uses`, which is emptied
  int settle(std::vector<Use> &uses)
  {
    for (Use &u : uses) {
      ACC_HIP_TRY(hipEventSynchronize(u.done));
      spare_events.push_back(u.done);
    }
    uses.clear();
    return ACC_OK;
  }

  // forget the uses that have completed; true if none is left
  bool idle(std::vector<Use> &uses)
  {
    for (size_t i = 0; i < uses.size();) {
      if (hipEventQuery(uses[i].done) == hipSuccess) {
        spare_events.push_back(uses[i].done);
        uses[i] = uses.back();
        uses.pop_back();
      } else {
        (void)hipGetLastError();   // hipErrorNotReady is not a failure
        ++i;
      }
    }
    return uses.empty();
  }

  void upload_settled(Entry &e)
  {
    if (e.uploaded) { spare_events.push_back(e.uploaded); e.uploaded = nullptr; }
  }

  int flush_nursery()
  {
    for (auto &kv : nursery) {
      ACC_TRY(settle(kv.second.uses));
      ACC_HIP_TRY(hipFree(kv.second.dev));
    }
    nursery.clear();
    st.nursery_bytes = 0;
    return ACC_OK;
  }

  // give up the device block of `e`: write back what only the device has, then
  // hand the block to the nursery (keep == true; work still reading it goes along
  // and is waited for when the block is reused) or to the device
  int drop(Entry &e, bool keep)
  {
    if (e.uploaded) { ACC_HIP_TRY(hipEventSynchronize(e.uploaded)); upload_settled(e); }
    if (e.status == DIRTY || !keep) ACC_TRY(settle(e.uses));
    if (e.status == DIRTY) {
      // (every use of the block has been waited for above: nothing the copy must be ordered behind)
      if (wants_staging(ctx, e.host, e.bytes)) ACC_TRY(staged_download(ctx, e.host, e.dev, e.bytes));
      else ACC_HIP_TRY(hipMemcpy(e.host, e.dev, e.bytes, hipMemcpyDeviceToHost));
      st.writebacks++;
      st.writeback_bytes += e.bytes;
    }
    st.resident_bytes -= e.rounded;
    st.resident_arrays--;
    if (keep) {
      FreeBlock fb;
      fb.dev = e.dev;
      fb.uses.swap(e.uses);
      nursery.emplace(e.rounded, std::move(fb));
      st.nursery_bytes += e.rounded;
    } else {
      ACC_HIP_TRY(hipFree(e.dev));
    }
    e.dev = nullptr;
    return ACC_OK;
  }

  // least recently used entry that may leave the device; nullptr if none.
  // Entries whose last use is still running are taken only when nothing idle is left.
  Entry *victim()
  {
    Entry *best = nullptr, *busy = nullptr;
    for (auto &kv : table) {
      Entry &e = kv.second;
      if (!e.dev || e.pins > 0 || e.status == UNMANAGED) continue;
      Entry *&slot = idle(e.uses) ? best : busy;
      if (!slot || e.tick < slot->tick) slot = &e;
    }
    return best ? best : busy;
  }

  int evict_one(bool *any)
  {
    Entry *v = victim();
    *any = v != nullptr;
    if (!v) return ACC_OK;
    Status after = (v->status == PENDING) ? PENDING : EVICTED;
    ACC_TRY(drop(*v, false));
    v->status = after;
    st.evictions++;
    return ACC_OK;
  }

  // a device block of `rounded` bytes: nursery, else the device; makes room first
  // when a budget says so and afterwards when the device says so
  int block(uint64_t rounded, void **out)
  {
    auto it = nursery.find(rounded);
    if (it != nursery.end()) {
      ACC_TRY(settle(it->second.uses));
      *out = it->second.dev;
      nursery.erase(it);
      st.nursery_bytes -= rounded;
      st.nursery_hits++;
      return ACC_OK;
    }
    if (budget && rounded > budget)
      return fail(ACC_ERR_OOM, "acc_memtable: an array of %llu bytes exceeds the table's budget of %llu",
                  (unsigned long long)rounded, (unsigned long long)budget);
    for (;;) {
      bool over = budget && held() + rounded > budget;
      if (!over) {
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, rounded);
        if (e == hipSuccess) { *out = p; st.device_allocs++; return ACC_OK; }
        (void)hipGetLastError();
        if (e != hipErrorOutOfMemory) return fail_hip(e, "hipMalloc");
      }
      if (!nursery.empty()) { ACC_TRY(flush_nursery()); continue; }
      // scratch the skeleton drivers are holding on to but not using (only worth anything against the device's
      // own limit: the budget counts arrays)
      if (!over && ctx->scratch_trim() > 0) continue;
      bool any = false;
      ACC_TRY(evict_one(&any));
      if (!any)
        return fail(ACC_ERR_OOM, "acc_memtable: %llu bytes do not fit and every resident array is in use "
                    "(%llu bytes resident%s)", (unsigned long long)rounded, (unsigned long long)st.resident_bytes,
                    budget ? ", budget reached" : "");
    }
  }
};

extern "C" {

int acc_memtable_create(acc_context ctx, uint64_t budget_bytes, acc_memtable *out)
{
  if (!ctx || !out) return fail(ACC_ERR_INVALID, "acc_memtable_create: NULL argument");
  *out = nullptr;
  ACC_TRY(ctx->make_current());
  acc_memtable mt = new acc_memtable_s();
  mt->ctx = ctx;
  mt->budget = budget_bytes;
  *out = mt;
  return ACC_OK;
}

int acc_memtable_destroy(acc_memtable mt)
{
  if (!mt) return ACC_OK;
  int rc = ACC_OK;
  {
    std::lock_guard<std::mutex> lock(mt->mu);
    rc = mt->ctx->make_current();
    if (rc == ACC_OK) {
      for (auto &kv : mt->table) {
        Entry &e = kv.second;
        (void)mt->settle(e.uses);
        if (e.uploaded) { (void)hipEventSynchronize(e.uploaded); mt->upload_settled(e); }
        if (e.dev && e.status != UNMANAGED) (void)hipFree(e.dev);
      }
      (void)mt->flush_nursery();
      for (hipEvent_t ev : mt->spare_events) (void)hipEventDestroy(ev);
    }
  }
  delete mt;
  return rc;
}

int acc_memtable_malloc(acc_memtable mt, uint64_t key, void *host, uint64_t bytes, int frozen, int *is_new)
{
  if (!mt) return fail(ACC_ERR_INVALID, "acc_memtable_malloc: NULL table");
  if (!host && bytes) return fail(ACC_ERR_INVALID, "acc_memtable_malloc: an array needs host storage to be evicted to");
  std::lock_guard<std::mutex> lock(mt->mu);
  ACC_TRY(mt->ctx->make_current());
  auto it = mt->table.find(key);
  if (it != mt->table.end()) {
    if (it->second.bytes != bytes)
      return fail(ACC_ERR_INVALID, "acc_memtable_malloc: key %llx is in the table with %llu bytes, not %llu",
                  (unsigned long long)key, (unsigned long long)it->second.bytes, (unsigned long long)bytes);
    if (is_new) *is_new = 0;
    return ACC_OK;
  }
  Entry e;
  e.host = host;
  e.bytes = bytes;
  e.rounded = round_up(bytes);
  e.frozen = frozen != 0;
  e.tick = ++mt->clock;
  if (frozen) {
    e.status = PENDING;       // the block is taken when the array is first wanted on the device
  } else {
    ACC_TRY(mt->block(e.rounded, &e.dev));
    e.status = DIRTY;
    mt->st.resident_bytes += e.rounded;
    mt->st.resident_arrays++;
  }
  mt->table.emplace(key, e);
  mt->st.arrays++;
  if (is_new) *is_new = 1;
  return ACC_OK;
}

int acc_memtable_acquire(acc_memtable mt, uint64_t key, acc_stream stream, acc_devptr *out)
{
  if (!mt || !out) return fail(ACC_ERR_INVALID, "acc_memtable_acquire: NULL argument");
  *out = 0;
  std::lock_guard<std::mutex> lock(mt->mu);
  ACC_TRY(mt->ctx->make_current());
  auto it = mt->table.find(key);
  if (it == mt->table.end())
    return fail(ACC_ERR_NOT_FOUND, "acc_memtable_acquire: key %llx is not in the table", (unsigned long long)key);
  Entry &e = it->second;
  if (e.status == EVICTED || e.status == PENDING) {
    if (!e.dev) {
      e.pins++;                               // never its own victim
      int rc = mt->block(e.rounded, &e.dev);
      e.pins--;
      if (rc != ACC_OK) return rc;
      mt->st.resident_bytes += e.rounded;
      mt->st.resident_arrays++;
    }
    if (e.bytes) {
      hipStream_t s = static_cast<hipStream_t>(stream);
      mt->upload_settled(e);
      ACC_TRY(mt->event(&e.uploaded));
      if (wants_staging(mt->ctx, e.host, e.bytes)) {
        // through the context's pinned buffers, on its copy stream: every stream that wants the array, this one
        // included, waits for the event recorded there (below)
        hipStream_t on = nullptr;
        ACC_TRY(staged_upload(mt->ctx, e.dev, e.host, e.bytes, nullptr, &on));
        ACC_HIP_TRY(hipEventRecord(e.uploaded, on));
        s = on;
      } else {
        ACC_HIP_TRY(hipMemcpyAsync(e.dev, e.host, e.bytes, hipMemcpyHostToDevice, s));
        ACC_HIP_TRY(hipEventRecord(e.uploaded, s));
      }
      e.upload_stream = s;
      mt->st.uploads++;
      mt->st.upload_bytes += e.bytes;
    }
    // what the device now holds is what the host holds; an array produced on the device is
    // taken to be changed again by whoever acquires it
    e.status = e.frozen ? CLEAN : DIRTY;
  }
  if (e.uploaded) {
    // an upload queued on another stream: this stream's work starts after it
    if (hipEventQuery(e.uploaded) == hipSuccess) {
      mt->upload_settled(e);
    } else {
      (void)hipGetLastError();
      if (e.upload_stream != static_cast<hipStream_t>(stream))
        ACC_HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(stream), e.uploaded, 0));
    }
  }
  e.pins++;
  e.tick = ++mt->clock;
  *out = reinterpret_cast<acc_devptr>(e.dev);
  return ACC_OK;
}

int acc_memtable_release(acc_memtable mt, uint64_t key, acc_stream stream)
{
  if (!mt) return fail(ACC_ERR_INVALID, "acc_memtable_release: NULL table");
  std::lock_guard<std::mutex> lock(mt->mu);
  ACC_TRY(mt->ctx->make_current());
  auto it = mt->table.find(key);
  if (it == mt->table.end())
    return fail(ACC_ERR_NOT_FOUND, "acc_memtable_release: key %llx is not in the table", (unsigned long long)key);
  Entry &e = it->second;
  if (e.pins <= 0) return fail(ACC_ERR_INVALID, "acc_memtable_release: key %llx is not acquired", (unsigned long long)key);
  if (e.status != UNMANAGED) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    Use *u = nullptr;
    for (Use &k : e.uses)
      if (k.stream == s) u = &k;
    if (!u) {
      mt->idle(e.uses);                  // keeps the list as short as the streams really in flight
      Use fresh;
      fresh.stream = s;
      ACC_TRY(mt->event(&fresh.done));
      e.uses.push_back(fresh);
      u = &e.uses.back();
    }
    ACC_HIP_TRY(hipEventRecord(u->done, s));
  }
  e.pins--;
  return ACC_OK;
}

int acc_memtable_free(acc_memtable mt, uint64_t key)
{
  if (!mt) return fail(ACC_ERR_INVALID, "acc_memtable_free: NULL table");
  std::lock_guard<std::mutex> lock(mt->mu);
  ACC_TRY(mt->ctx->make_current());
  auto it = mt->table.find(key);
  if (it == mt->table.end()) return ACC_OK;       // freeing twice is harmless (Array/Remote.hs:166-168)
  Entry &e = it->second;
  if (e.pins > 0) return fail(ACC_ERR_INVALID, "acc_memtable_free: key %llx is still acquired", (unsigned long long)key);
  if (e.dev && e.status != UNMANAGED) {
    e.status = CLEAN;                              // nobody will read it: nothing to write back
    ACC_TRY(mt->drop(e, true));
    if (mt->budget && mt->held() > mt->budget) ACC_TRY(mt->flush_nursery());
  }
  ACC_TRY(mt->settle(e.uses));            // (empty when the block went to the nursery with them)
  if (e.uploaded) { ACC_HIP_TRY(hipEventSynchronize(e.uploaded)); mt->upload_settled(e); }
  mt->table.erase(it);
  mt->st.arrays--;
  return ACC_OK;
}

int acc_memtable_insert_unmanaged(acc_memtable mt, uint64_t key, acc_devptr p, uint64_t bytes)
{
  if (!mt || !p) return fail(ACC_ERR_INVALID, "acc_memtable_insert_unmanaged: NULL argument");
  std::lock_guard<std::mutex> lock(mt->mu);
  if (mt->table.count(key))
    return fail(ACC_ERR_INVALID, "acc_memtable_insert_unmanaged: key %llx is already in the table", (unsigned long long)key);
  Entry e;
  e.bytes = bytes;
  e.rounded = 0;                                   // not counted: the table does not hold it
  e.dev = reinterpret_cast<void *>(p);
  e.status = UNMANAGED;
  e.tick = ++mt->clock;
  mt->table.emplace(key, e);
  mt->st.arrays++;
  return ACC_OK;
}

int acc_memtable_reclaim(acc_memtable mt)
{
  if (!mt) return fail(ACC_ERR_INVALID, "acc_memtable_reclaim: NULL table");
  std::lock_guard<std::mutex> lock(mt->mu);
  ACC_TRY(mt->ctx->make_current());
  return mt->flush_nursery();
}

int acc_memtable_get_stats(acc_memtable mt, acc_memtable_stats *out)
{
  if (!mt || !out) return fail(ACC_ERR_INVALID, "acc_memtable_get_stats: NULL argument");
  std::lock_guard<std::mutex> lock(mt->mu);
  *out = mt->st;
  return ACC_OK;
}

}  // extern "C"
