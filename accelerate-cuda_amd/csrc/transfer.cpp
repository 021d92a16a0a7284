// Transfers between pageable host memory and the device at the speed of the link.
//
// The reference moves every operand and every result of `run` through pokeArray / peekArray (Array/Prim.hs:189-234,
// Execute.hs:146-154, CUDA.hs:382-389), from and to ordinary Haskell heap arrays.  A copy from pageable memory is
// staged by the runtime through a bounce buffer of its own, one piece after the other: about 15 GB/s here, a quarter
// of what the link carries.  This file stages such copies itself: the source is cut into chunks, a few threads copy
// a chunk into one of a ring of pinned buffers while the copy engine moves the chunks before it (and the other way
// round for results), so that the host's copying and the link's work overlap.  Memory that exists is never
// registered with the runtime; the pinned buffers are allocated as such.
#include <algorithm>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <thread>

#include "acc_internal.hpp"

namespace acc {

class Stager {
 public:
  static constexpr size_t CHUNK = size_t(4) << 20;
  static constexpr int RING = 8;

  explicit Stager(int helpers) : helpers_(std::max(0, std::min(helpers, 15))) {}

  ~Stager()
  {
    {
      std::lock_guard<std::mutex> lock(qmu_);
      stop_ = true;
    }
    qcv_.notify_all();
    for (std::thread &t : threads_) t.join();
    for (int b = 0; b < RING; ++b) {
      if (ev_[b]) (void)hipEventDestroy(ev_[b]);
      if (pinned_[b]) (void)hipHostFree(pinned_[b]);
    }
    if (stream_) (void)hipStreamDestroy(stream_);
  }

  // host -> device.  Returns when every chunk has been handed to the copy engine on the stager's stream; *done (an
  // event of the stager's, valid until its next transfer) is recorded behind the last one.
  int h2d(void *dev, const void *host, size_t bytes, hipEvent_t *done)
  {
    std::lock_guard<std::mutex> lock(mu_);
    ACC_TRY(setup());
    const char *src = static_cast<const char *>(host);
    char *dst = static_cast<char *>(dev);
    int i = 0;
    for (size_t off = 0; off < bytes; off += CHUNK, ++i) {
      const int b = i % RING;
      const size_t n = std::min(CHUNK, bytes - off);
      if (used_[b]) ACC_HIP_TRY(hipEventSynchronize(ev_[b]));      // the engine has read what the buffer held
      parallel_copy(pinned_[b], src + off, n);
      ACC_HIP_TRY(hipMemcpyAsync(dst + off, pinned_[b], n, hipMemcpyHostToDevice, stream_));
      ACC_HIP_TRY(hipEventRecord(ev_[b], stream_));
      used_[b] = true;
    }
    ACC_HIP_TRY(hipEventRecord(all_, stream_));
    if (done) *done = all_;
    return ACC_OK;
  }

  // device -> host; returns when the data is in `host`.  The caller has made sure that what produces `dev` is done.
  int d2h(void *host, const void *dev, size_t bytes)
  {
    std::lock_guard<std::mutex> lock(mu_);
    ACC_TRY(setup());
    char *dst = static_cast<char *>(host);
    const char *src = static_cast<const char *>(dev);
    const size_t chunks = (bytes + CHUNK - 1) / CHUNK;
    auto issue = [&](size_t c) -> int {
      const int b = static_cast<int>(c % RING);
      const size_t off = c * CHUNK, n = std::min(CHUNK, bytes - off);
      ACC_HIP_TRY(hipMemcpyAsync(pinned_[b], src + off, n, hipMemcpyDeviceToHost, stream_));
      ACC_HIP_TRY(hipEventRecord(ev_[b], stream_));
      used_[b] = true;
      return ACC_OK;
    };
    for (int b = 0; b < RING; ++b)
      if (used_[b]) ACC_HIP_TRY(hipEventSynchronize(ev_[b]));      // (an upload may still be reading the ring)
    for (size_t c = 0; c < std::min<size_t>(chunks, RING); ++c) ACC_TRY(issue(c));
    for (size_t c = 0; c < chunks; ++c) {
      const int b = static_cast<int>(c % RING);
      const size_t off = c * CHUNK, n = std::min(CHUNK, bytes - off);
      ACC_HIP_TRY(hipEventSynchronize(ev_[b]));
      parallel_copy(dst + off, pinned_[b], n);
      if (c + RING < chunks) ACC_TRY(issue(c + RING));
    }
    return ACC_OK;
  }

  int wait()                                // everything handed to the engine so far has been moved
  {
    std::lock_guard<std::mutex> lock(mu_);
    if (!stream_) return ACC_OK;
    ACC_HIP_TRY(hipStreamSynchronize(stream_));
    return ACC_OK;
  }

  hipStream_t stream() const { return stream_; }

 private:
  struct Task { void *dst; const void *src; size_t n; };

  int setup()
  {
    if (ready_) return ACC_OK;
    if (!stream_) ACC_HIP_TRY(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));     // default priority
    if (!all_) ACC_HIP_TRY(hipEventCreateWithFlags(&all_, hipEventDisableTiming));
    for (int b = 0; b < RING; ++b) {
      if (!pinned_[b]) ACC_HIP_TRY(hipHostMalloc(&pinned_[b], CHUNK, hipHostMallocDefault));
      if (!ev_[b]) ACC_HIP_TRY(hipEventCreateWithFlags(&ev_[b], hipEventDisableTiming));
    }
    for (int t = static_cast<int>(threads_.size()); t < helpers_; ++t) threads_.emplace_back([this] { work(); });
    ready_ = true;
    return ACC_OK;
  }

  // the calling thread and the helpers copy a share each
  void parallel_copy(void *dst, const void *src, size_t n)
  {
    const size_t parts = static_cast<size_t>(helpers_) + 1;
    const size_t share = ((n + parts - 1) / parts + 4095) & ~size_t(4095);
    size_t first = std::min(share, n);
    if (helpers_ > 0 && n > first) {
      std::lock_guard<std::mutex> lock(qmu_);
      for (size_t off = first; off < n; off += share) {
        queue_.push_back(Task{static_cast<char *>(dst) + off, static_cast<const char *>(src) + off, std::min(share, n - off)});
        ++outstanding_;
      }
      qcv_.notify_all();
    } else {
      first = n;
    }
    std::memcpy(dst, src, first);
    std::unique_lock<std::mutex> lock(qmu_);
    dcv_.wait(lock, [&] { return outstanding_ == 0; });
  }

  void work()
  {
    for (;;) {
      Task t;
      {
        std::unique_lock<std::mutex> lock(qmu_);
        qcv_.wait(lock, [&] { return stop_ || !queue_.empty(); });
        if (stop_) return;
        t = queue_.front();
        queue_.pop_front();
      }
      std::memcpy(t.dst, t.src, t.n);
      {
        std::lock_guard<std::mutex> lock(qmu_);
        if (--outstanding_ == 0) dcv_.notify_all();
      }
    }
  }

  const int helpers_;
  std::mutex mu_;                 // one staged transfer at a time
  bool ready_ = false;
  hipStream_t stream_ = nullptr;
  hipEvent_t all_ = nullptr;
  void *pinned_[RING] = {};
  hipEvent_t ev_[RING] = {};
  bool used_[RING] = {};
  std::mutex qmu_;
  std::condition_variable qcv_, dcv_;
  std::deque<Task> queue_;
  size_t outstanding_ = 0;
  bool stop_ = false;
  std::vector<std::thread> threads_;
};

// ---- the context's side ---------------------------------------------------------

static Stager *stager_of(acc_context ctx)
{
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (!ctx->stager) ctx->stager = new Stager(ctx->copy_helpers);
  return ctx->stager;
}

void stager_destroy(acc_context ctx)
{
  Stager *s = nullptr;
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    s = ctx->stager;
    ctx->stager = nullptr;
  }
  delete s;
}

// is a copy of `bytes` bytes from / to `host` one for the stager?  Large, and in memory the runtime does not know
// (pinned memory goes to the copy engine as it is)
bool wants_staging(acc_context ctx, const void *host, size_t bytes)
{
  if (bytes < ctx->copy_staged_from) return false;
  hipPointerAttribute_t attr;
  const hipError_t e = hipPointerGetAttributes(&attr, host);
  if (e != hipSuccess) {
    (void)hipGetLastError();                 // an address the runtime has never seen: pageable
    return true;
  }
  return attr.type == hipMemoryTypeUnregistered;
}

int staged_upload(acc_context ctx, void *dev, const void *host, size_t bytes, hipEvent_t *done, hipStream_t *on)
{
  Stager *s = stager_of(ctx);
  ACC_TRY(s->h2d(dev, host, bytes, done));
  if (on) *on = s->stream();
  return ACC_OK;
}

int staged_upload_wait(acc_context ctx) { return stager_of(ctx)->wait(); }

int staged_download(acc_context ctx, void *host, const void *dev, size_t bytes) { return stager_of(ctx)->d2h(host, dev, bytes); }

}  // namespace acc
