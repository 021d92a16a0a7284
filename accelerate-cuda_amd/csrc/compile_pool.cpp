// Run-time compilation in the background.
//
// The reference compiles on forked threads, no more at a time than the machine has processors, while its main
// thread goes on generating code, and blocks only where a kernel is first used (Compile.hs:444-459 `link`, :484-538
// `build1`, :620-660 `enqueueProcess` / `workers`): that is why a program's kernels take as long to get ready as the
// slowest of them, not as all of them together.  Here the compiler is hiprtc and the pool is a set of threads started
// as jobs arrive, each with a helper process of its own to compile in (compile_child.cpp: hiprtc takes one program at
// a time per process).  A job holds copies of all the compiler reads; whoever needs its code waits for it
// (acc_skel_s::ensure_variant), and gets the worker's error text and compile log as if it had compiled itself.
#include <algorithm>
#include <cstdlib>
#include <deque>
#include <thread>

#include "acc_internal.hpp"

namespace acc {

void CompileJob::run()
{
  std::vector<const char *> optp;
  for (const std::string &o : options) optp.push_back(o.c_str());
  const void *c = nullptr;
  size_t n = 0;
  const int r = acc_compile(nullptr, target.c_str(), source.c_str(), optp.data(), static_cast<int>(optp.size()), &c, &n);
  std::string err = r == ACC_OK ? std::string() : last_error_text();
  std::string lg = compile_log_text();
  {
    std::lock_guard<std::mutex> lock(mu);
    rc = r;
    error = std::move(err);
    log = std::move(lg);
    code = c;
    size = n;
    done = true;
  }
  cv.notify_all();
}

int CompileJob::wait()
{
  std::unique_lock<std::mutex> lock(mu);
  cv.wait(lock, [&] { return done; });
  set_compile_log(log);
  if (rc != ACC_OK) set_last_error(error);
  return rc;
}

namespace {

// The pool lives until the process ends.  A worker that is still inside the compiler when exit() starts tearing down
// static data -- the compiler's own among it, some of it created in the middle of a compilation and therefore torn
// down BEFORE this pool -- crashes the process on its way out; so a host calls acc_compile_drain before it exits
// (the Python binding registers it with `atexit`, the Haskell one registers the C function with the C library's).  The destructor does the
// same for what is left, which is too late only for a compilation in flight at that moment.
class Pool {
 public:
  ~Pool() { drain(); }

  // No compilation runs or starts after this: what is queued is abandoned (whoever waits for it gets an error), the
  // workers finish the job they have in hand and end.  For the end of the process.
  void drain()
  {
    std::vector<std::thread> ending;
    {
      std::lock_guard<std::mutex> lock(mu_);
      stop_ = true;
      for (auto &j : queue_) abandon(j);
      queue_.clear();
      ending.swap(workers_);
    }
    cv_.notify_all();
    for (std::thread &t : ending) t.join();
  }

  bool submit(const std::shared_ptr<CompileJob> &job)
  {
    {
      std::lock_guard<std::mutex> lock(mu_);
      if (stop_) return false;              // drained: the caller compiles on its own thread
      queue_.push_back(job);
      // one more worker while more jobs wait than workers do, and the bound allows
      if (static_cast<int>(queue_.size()) > idle_ && static_cast<int>(workers_.size()) < limit()) workers_.emplace_back([this] { work(); });
    }
    cv_.notify_one();
    return true;
  }

  static int limit()
  {
    // as many as the machine has processors (Compile.hs:629 getNumProcessors), at most 16 unless
    // ACC_HIP_COMPILE_THREADS says otherwise (a container often sees more processors than it may use)
    static const int n = [] {
      int want = static_cast<int>(std::thread::hardware_concurrency());
      if (want < 1) want = 1;
      want = std::min(want, 16);
      if (const char *e = std::getenv("ACC_HIP_COMPILE_THREADS")) {
        const int v = std::atoi(e);
        if (v >= 1 && v <= 256) want = v;
      }
      return want;
    }();
    return n;
  }

 private:
  static void abandon(const std::shared_ptr<CompileJob> &job)
  {
    {
      std::lock_guard<std::mutex> lock(job->mu);
      job->rc = ACC_ERR_COMPILE;
      job->error = "run-time compilation abandoned: the process is ending";
      job->done = true;
    }
    job->cv.notify_all();
  }

  void work()
  {
    compile_child_attach();                 // this thread's compilations run in a helper process of its own
    struct Detach { ~Detach() { compile_child_detach(); } } detach;
    for (;;) {
      std::shared_ptr<CompileJob> job;
      {
        std::unique_lock<std::mutex> lock(mu_);
        ++idle_;
        cv_.wait(lock, [&] { return stop_ || !queue_.empty(); });
        --idle_;
        if (stop_) return;
        job = queue_.front();
        queue_.pop_front();
      }
      job->run();
    }
  }

  std::mutex mu_;
  std::condition_variable cv_;
  std::deque<std::shared_ptr<CompileJob>> queue_;
  std::vector<std::thread> workers_;
  int idle_ = 0;
  bool stop_ = false;
};

Pool &pool()
{
  static Pool p;
  return p;
}

}  // namespace

bool compile_submit(const std::shared_ptr<CompileJob> &job) { return pool().submit(job); }
void compile_drain() { pool().drain(); }
int compile_pool_threads() { return Pool::limit(); }

}  // namespace acc
