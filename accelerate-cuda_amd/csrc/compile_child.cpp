// Compilation in processes of their own.
//
// hiprtc compiles one program at a time per process, however many threads ask.  The reference compiles a program's
// kernels side by side because its compiler is a process of its own, forked once per kernel (Compile.hs:543-594:
// `nvcc` through createProcess, as many at a time as the machine has processors); here every thread of the worker
// pool keeps one helper process -- lib/acc_compile_worker, a few lines of main() over this library -- hands it the
// source, the target and the options over a socket pair and gets the code object and the compiler's log back.  The
// helper never touches the device.  Where the helper cannot be started (the library was linked into a program, the
// file is gone) the thread compiles in process as before.
#include <dlfcn.h>
#include <spawn.h>
#include <sys/socket.h>
#include <sys/wait.h>
#include <unistd.h>

#include <cerrno>
#include <cstdlib>
#include <cstring>

#include "acc_internal.hpp"

extern char **environ;

namespace acc {
namespace {

constexpr uint32_t kMagic = 0xACC1C0DEu;

bool send_all(int fd, const void *p, size_t n)
{
  const char *c = static_cast<const char *>(p);
  while (n > 0) {
    const ssize_t k = ::send(fd, c, n, MSG_NOSIGNAL);
    if (k < 0 && errno == EINTR) continue;
    if (k <= 0) return false;
    c += k;
    n -= static_cast<size_t>(k);
  }
  return true;
}

bool recv_all(int fd, void *p, size_t n)
{
  char *c = static_cast<char *>(p);
  while (n > 0) {
    const ssize_t k = ::recv(fd, c, n, 0);
    if (k < 0 && errno == EINTR) continue;
    if (k <= 0) return false;
    c += k;
    n -= static_cast<size_t>(k);
  }
  return true;
}

bool send_text(int fd, const std::string &s)
{
  const uint64_t n = s.size();
  return send_all(fd, &n, 8) && (n == 0 || send_all(fd, s.data(), n));
}

bool recv_text(int fd, std::string *s, uint64_t limit)
{
  uint64_t n = 0;
  if (!recv_all(fd, &n, 8) || n > limit) return false;
  s->resize(n);
  return n == 0 || recv_all(fd, &(*s)[0], n);
}

std::string worker_path()
{
  Dl_info info;
  if (!dladdr(reinterpret_cast<void *>(&acc_compile), &info) || !info.dli_fname) return std::string();
  std::string p = info.dli_fname;
  const size_t slash = p.rfind('/');
  if (slash == std::string::npos) return std::string();
  p.resize(slash + 1);
  p += "acc_compile_worker";
  return access(p.c_str(), X_OK) == 0 ? p : std::string();
}

}  // namespace

struct CompilerChild {
  int fd = -1;
  pid_t pid = -1;
  bool failed = false;      // could not be started, or died: this thread compiles in process from now on

  ~CompilerChild() { stop(); }

  void stop()
  {
    if (fd >= 0) { ::close(fd); fd = -1; }                 // the helper sees the end of its input and leaves
    if (pid > 0) { int st = 0; (void)waitpid(pid, &st, 0); pid = -1; }
  }

  bool start()
  {
    static const std::string path = worker_path();
    if (path.empty()) return false;
    int sv[2];
    if (socketpair(AF_UNIX, SOCK_STREAM | SOCK_CLOEXEC, 0, sv) != 0) return false;
    posix_spawn_file_actions_t fa;
    posix_spawn_file_actions_init(&fa);
    posix_spawn_file_actions_adddup2(&fa, sv[1], 0);       // the helper talks over its descriptor 0, both ways
    char *const argv[] = {const_cast<char *>(path.c_str()), nullptr};
    pid_t child = -1;
    const int rc = posix_spawn(&child, path.c_str(), &fa, nullptr, argv, environ);
    posix_spawn_file_actions_destroy(&fa);
    ::close(sv[1]);
    if (rc != 0) { ::close(sv[0]); return false; }
    fd = sv[0];
    pid = child;
    return true;
  }

  // true: the helper answered (rc, log and code are its answer); false: it could not be reached
  bool compile(const std::string &target, const char *source, const std::vector<std::string> &options, std::vector<char> *code,
               std::string *log, int *rc)
  {
    if (failed) return false;
    if (fd < 0 && !start()) { failed = true; return false; }
    const uint32_t head[2] = {kMagic, static_cast<uint32_t>(options.size())};
    bool ok = send_all(fd, head, sizeof(head)) && send_text(fd, target);
    for (size_t i = 0; ok && i < options.size(); ++i) ok = send_text(fd, options[i]);
    ok = ok && send_text(fd, source);
    int32_t status = 0;
    std::string text;
    ok = ok && recv_all(fd, &status, 4) && recv_text(fd, log, 64u << 20) && recv_text(fd, &text, 1ull << 30);
    if (!ok) { stop(); failed = true; return false; }
    code->assign(text.begin(), text.end());
    *rc = status;
    return true;
  }
};

static thread_local CompilerChild *t_child = nullptr;

// a worker thread of the pool: its compilations go to a helper process from now on
void compile_child_attach()
{
  static const bool enabled = [] {
    const char *e = std::getenv("ACC_HIP_COMPILE_PROCESSES");      // 0: compile in process (one at a time)
    return !(e && std::atoi(e) == 0 && *e);
  }();
  if (enabled && !t_child) t_child = new CompilerChild();
}

void compile_child_detach()
{
  delete t_child;
  t_child = nullptr;
}

bool compile_out_of_process(const std::string &target, const char *source, const std::vector<std::string> &options,
                            std::vector<char> *code, std::string *log, int *rc)
{
  return t_child && t_child->compile(target, source, options, code, log, rc);
}

}  // namespace acc

// the helper's whole main(): requests from descriptor `fd` until it closes
extern "C" __attribute__((visibility("default"))) int acc_compile_worker_main(int fd)
{
  using namespace acc;
  for (;;) {
    uint32_t head[2];
    if (!recv_all(fd, head, sizeof(head))) return 0;               // the library has gone
    if (head[0] != kMagic || head[1] > 256) return 2;
    std::string target, source;
    std::vector<std::string> options(head[1]);
    if (!recv_text(fd, &target, 256)) return 2;
    for (std::string &o : options)
      if (!recv_text(fd, &o, 1 << 20)) return 2;
    if (!recv_text(fd, &source, 1ull << 30)) return 2;
    std::vector<char> code;
    const int32_t rc = compile_in_process(target, source.c_str(), options, &code);
    const std::string log = compile_log_text();
    if (!send_all(fd, &rc, 4) || !send_text(fd, log) || !send_text(fd, std::string(code.begin(), code.end()))) return 2;
  }
}
